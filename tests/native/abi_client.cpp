// A C++ caller of libyka.so that uses nothing but include/yka_abi.h and the HIP runtime - the shape of the call site a
// maintainer of the reference engine would write inside attn_block (engine35.cpp:882-951): device buffers owned by the
// caller, the position on the device, one stream, append + attention per layer call, a captured pass replayed at a
// new position.  Exits 0 and prints "abi_client ok" when every check holds.
#include "yka_abi.h"
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); return 1; } } while (0)
#define YKA_OK(x) do { if ((x) != 0) { std::printf("yka error at line %d: %s\n", __LINE__, yka_last_error()); return 1; } } while (0)
#define CHECK(c) do { if (!(c)) { std::printf("check failed at line %d: %s\n", __LINE__, #c); return 1; } } while (0)

// fp16 bit patterns of small pseudo-random values in (-2, 2): sign, exponent 12..15, 10 mantissa bits
static uint16_t rnd16(uint32_t& s) {
  s = s * 1664525u + 1013904223u;
  const uint32_t r = s >> 8;
  return (uint16_t)(((r & 1u) << 15) | ((12u + ((r >> 1) & 3u)) << 10) | ((r >> 3) & 0x3ffu));
}

int main() {
  const int NH = 24, KVH = 4, D = 128, CTX = 700, M = 5, MAXCTX = 1024;
  std::printf("%s\n", yka_build_info());

  yka_kv_config cfg{};
  cfg.n_layers = 2; cfg.n_heads = NH; cfg.n_kv_heads = KVH; cfg.head_dim = D; cfg.max_ctx = MAXCTX; cfg.max_rows = 64;
  cfg.paged = 0; cfg.device = 0;
  yka_kv* kv = yka_kv_open(&cfg);
  if (!kv) { std::printf("open failed: %s\n", yka_last_error()); return 1; }

  // error convention: -1 and a message, the handle stays usable
  CHECK(yka_attend(kv, 7, nullptr, 1, nullptr, nullptr, nullptr, nullptr) == -1);
  CHECK(std::strlen(yka_last_error()) > 0);
  yka_kv_config bad = cfg; bad.head_dim = 64;
  CHECK(yka_kv_open(&bad) == nullptr);

  uint32_t seed = 12345u;
  std::vector<uint16_t> k((size_t)(CTX + 2 * M) * KVH * D), v(k.size()), q((size_t)M * NH * D), q2(q.size());
  for (auto& x : k) x = rnd16(seed);
  for (auto& x : v) x = rnd16(seed);
  for (auto& x : q) x = rnd16(seed);
  for (auto& x : q2) x = rnd16(seed);

  // the cached part, in chunks of at most max_rows, into both containers
  for (int layer = 0; layer < 2; ++layer)
    for (int p = 0; p < CTX; p += 64) {
      const int n = CTX - p < 64 ? CTX - p : 64;
      YKA_OK(yka_append_host(kv, layer, k.data() + (size_t)p * KVH * D, v.data() + (size_t)p * KVH * D, n, p));
    }

  // layer call with device pointers on the caller's stream (container 0)
  hipStream_t st; HIP_OK(hipStreamCreate(&st));
  uint16_t *dq, *dk, *dv, *dout; int* dpos;
  const size_t nq = (size_t)M * NH * D, nk = (size_t)M * KVH * D;
  HIP_OK(hipMalloc(&dq, nq * 2)); HIP_OK(hipMalloc(&dk, nk * 2)); HIP_OK(hipMalloc(&dv, nk * 2)); HIP_OK(hipMalloc(&dout, nq * 2));
  HIP_OK(hipMalloc(&dpos, sizeof(int)));
  const uint16_t* knew = k.data() + (size_t)CTX * KVH * D; const uint16_t* vnew = v.data() + (size_t)CTX * KVH * D;
  int pos = CTX;
  HIP_OK(hipMemcpyAsync(dq, q.data(), nq * 2, hipMemcpyHostToDevice, st));
  HIP_OK(hipMemcpyAsync(dk, knew, nk * 2, hipMemcpyHostToDevice, st));
  HIP_OK(hipMemcpyAsync(dv, vnew, nk * 2, hipMemcpyHostToDevice, st));
  HIP_OK(hipMemcpyAsync(dpos, &pos, sizeof(int), hipMemcpyHostToDevice, st));
  YKA_OK(yka_append_attend(kv, 0, dq, dk, dv, M, dpos, nullptr, dout, st));
  std::vector<uint16_t> out_dev(nq), out_host(nq), out_graph(nq), out_host2(nq);
  HIP_OK(hipMemcpyAsync(out_dev.data(), dout, nq * 2, hipMemcpyDeviceToHost, st));
  HIP_OK(hipStreamSynchronize(st));

  // the same call through the host-pointer hook on container 1: same kernels, same split counts -> same bits
  YKA_OK(yka_layer_call_host(kv, 1, q.data(), knew, vnew, M, CTX, nullptr, out_host.data()));
  CHECK(std::memcmp(out_dev.data(), out_host.data(), nq * 2) == 0);
  bool nonzero = false;
  for (uint16_t x : out_dev) nonzero |= (x & 0x7fffu) != 0;
  CHECK(nonzero);

  // both containers now hold the same rows
  std::vector<uint8_t> kc0((size_t)KVH * M * 64), vc0(kc0.size()), kc1(kc0.size()), vc1(kc0.size());
  std::vector<uint16_t> ks0((size_t)KVH * M * 4), vs0(ks0.size()), ks1(ks0.size()), vs1(ks0.size());
  YKA_OK(yka_kv_export_rows(kv, 0, CTX, M, kc0.data(), ks0.data(), vc0.data(), vs0.data()));
  YKA_OK(yka_kv_export_rows(kv, 1, CTX, M, kc1.data(), ks1.data(), vc1.data(), vs1.data()));
  CHECK(kc0 == kc1 && vc0 == vc1 && ks0 == ks1 && vs0 == vs1);

  // a captured pass over container 0, replayed at the next position with new rows: only device memory changes
  int32_t layers[1] = {0};
  yka_pass* pass = yka_pass_capture(kv, layers, 1, dq, dk, dv, M, dpos, nullptr, dout, 0);
  if (!pass) { std::printf("capture failed: %s\n", yka_last_error()); return 1; }
  const uint16_t* knew2 = k.data() + (size_t)(CTX + M) * KVH * D; const uint16_t* vnew2 = v.data() + (size_t)(CTX + M) * KVH * D;
  pos = CTX + M;
  HIP_OK(hipMemcpyAsync(dq, q2.data(), nq * 2, hipMemcpyHostToDevice, st));
  HIP_OK(hipMemcpyAsync(dk, knew2, nk * 2, hipMemcpyHostToDevice, st));
  HIP_OK(hipMemcpyAsync(dv, vnew2, nk * 2, hipMemcpyHostToDevice, st));
  HIP_OK(hipMemcpyAsync(dpos, &pos, sizeof(int), hipMemcpyHostToDevice, st));
  YKA_OK(yka_pass_launch(pass, st));
  HIP_OK(hipMemcpyAsync(out_graph.data(), dout, nq * 2, hipMemcpyDeviceToHost, st));
  HIP_OK(hipStreamSynchronize(st));
  YKA_OK(yka_layer_call_host(kv, 1, q2.data(), knew2, vnew2, M, CTX + M, nullptr, out_host2.data()));
  CHECK(std::memcmp(out_graph.data(), out_host2.data(), nq * 2) == 0);
  CHECK(std::memcmp(out_graph.data(), out_dev.data(), nq * 2) != 0);
  yka_pass_destroy(pass);

  HIP_OK(hipFree(dq)); HIP_OK(hipFree(dk)); HIP_OK(hipFree(dv)); HIP_OK(hipFree(dout)); HIP_OK(hipFree(dpos));
  HIP_OK(hipStreamDestroy(st));
  yka_kv_close(kv);
  std::printf("abi_client ok\n");
  return 0;
}
