// The selector memo of the C++ scheduler mirror on the GPU: three tensors whose
// entries are -1 (a dense one, a ReLU-like one, a tiny one) are walked for several
// iterations.  The first iteration probes; the following ones reuse a remembered
// ZFP / raw decision without a probe (cswap_engine_probe_count does not move for
// them), the ZVC tensor is probed every time, and after `recheck` reuses a
// remembered decision is probed again.  Built and run by tests/test_gpu_execution.py;
// prints "OK <probes per iteration...>" on success.
#include <hip/hip_runtime_api.h>
#include <stdio.h>
#include <string.h>

#include <vector>

#include "cswap_execution.hpp"

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("hip error %d at line %d\n", (int)e_, __LINE__); return 2; } } while (0)
#define CS_OK(x) do { int r_ = (x); if (r_ != CSWAP_OK) { printf("cswap error %d (%s) at line %d\n", r_, cswap_strerror(r_), __LINE__); return 3; } } while (0)

int main()
{
  struct Shape { size_t nx, ny, nz; };
  const Shape shapes[3] = {{32, 32, 4096}, {32, 32, 4096}, {8, 8, 16}};  // 16 MiB dense, 16 MiB ReLU-like, 4 KiB
  cswap_engine_config cfg;
  cswap_engine_config_default(&cfg);
  cfg.pinned_pool_bytes = (size_t)128 << 20;
  cfg.device_pool_bytes = (size_t)128 << 20;
  cswap_engine* eng = nullptr;
  CS_OK(cswap_engine_create(&eng, &cfg));

  std::vector<std::vector<float>> host(3);
  float* dev[3];
  unsigned s = 2024;
  for (int i = 0; i < 3; i++) {
    const size_t n = shapes[i].nx * shapes[i].ny * shapes[i].nz;
    host[(size_t)i].resize(n);
    for (size_t k = 0; k < n; k++) {
      s = s * 1664525u + 1013904223u;
      float v = (float)((s >> 8) & 0xffff) / 65536.0f - 0.5f;
      if (i == 1 && ((s >> 24) % 10) < 7) v = 0.0f;
      host[(size_t)i][k] = v;
    }
    HIP_OK(hipMalloc((void**)&dev[i], 4 * n));
    HIP_OK(hipMemcpy(dev[i], host[(size_t)i].data(), 4 * n, hipMemcpyHostToDevice));
  }
  hipStream_t compute;
  HIP_OK(hipStreamCreate(&compute));

  cswap::Execution exe(eng);
  exe.init_(4);
  exe.policy = {-1, -1, -1, 0};
  exe.recheck = 2;
  std::vector<float> back;
  int tags[3] = {0, 0, 0};
  std::vector<unsigned long long> probes;
  for (int iter = 0; iter < 5; iter++) {
    const unsigned long long before = cswap_engine_probe_count(eng);
    exe.preforward();
    CS_OK(exe.pre(-1, nullptr, 1, 1, 1, compute));  // op 0 produces tensor 0
    exe.post();
    for (int i = 0; i < 3; i++) {                   // op i+1 consumes tensor i
      CS_OK(exe.pre(i, dev[i], shapes[i].nx, shapes[i].ny, shapes[i].nz, compute));
      int st = 0;
      exe.post(&st);
      CS_OK(st);
    }
    exe.postforward();
    probes.push_back(cswap_engine_probe_count(eng) - before);
    for (int i = 2; i >= 0; i--) {
      const size_t n = host[(size_t)i].size();
      const int tag = exe.com_and_tran(i);
      if (iter == 0) tags[i] = tag;
      if (tag != tags[i]) { printf("iteration %d tensor %d: tag %d, was %d\n", iter, i, tag, tags[i]); return 4; }
      HIP_OK(hipMemsetAsync(dev[i], 0xff, 4 * n, compute));
      CS_OK(exe.fetch(i, dev[i], compute));
      HIP_OK(hipStreamSynchronize(compute));
      back.resize(n);
      HIP_OK(hipMemcpy(back.data(), dev[i], 4 * n, hipMemcpyDeviceToHost));
      if (tag != CSWAP_POLICY_ZFP) {
        if (memcmp(back.data(), host[(size_t)i].data(), 4 * n) != 0) { printf("tensor %d came back different\n", i); return 5; }
      } else {
        for (size_t k = 0; k < n; k++)
          if (!(back[k] - host[(size_t)i][k] < 0.1f && host[(size_t)i][k] - back[k] < 0.1f)) { printf("tensor %d value %zu off\n", i, k); return 5; }
        HIP_OK(hipMemcpy(dev[i], host[(size_t)i].data(), 4 * n, hipMemcpyHostToDevice));  // the lossless input again
      }
    }
  }
  // dense -> ZFP, ReLU-like -> ZVC, tiny -> raw (not even probed: it cannot pay for it)
  if (tags[0] != CSWAP_POLICY_ZFP || tags[1] != CSWAP_POLICY_SPARSE || tags[2] != CSWAP_POLICY_NONE) {
    printf("tags %d %d %d\n", tags[0], tags[1], tags[2]);
    return 6;
  }
  // iteration 0: dense + ReLU probed; 1 and 2: the ReLU tensor only; 3: the memo has been
  // used `recheck` times, the dense tensor is probed again; 4: reused again
  const unsigned long long want[5] = {2, 1, 1, 2, 1};
  for (int i = 0; i < 5; i++)
    if (probes[(size_t)i] != want[i]) { printf("iteration %d: %llu probes, expected %llu\n", i, probes[(size_t)i], want[i]); return 7; }
  if (exe.memo_hits != 2 * 3) { printf("memo hits %ld\n", exe.memo_hits); return 8; }
  for (int i = 0; i < 3; i++) HIP_OK(hipFree(dev[i]));
  HIP_OK(hipStreamDestroy(compute));
  cswap_engine_destroy(eng);
  printf("OK");
  for (unsigned long long p : probes) printf(" %llu", p);
  printf("\n");
  return 0;
}
