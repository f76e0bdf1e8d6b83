// Throughput of fp32 global atomic adds on gfx950, in the pattern a single-pass backward would
// need: every (query tile, key tile) pair adds a [32 keys x 128] fp32 partial of dk (and one of
// dv) into global memory, as the upstream kernel does under its spin lock
// (stickbreaking_attention/sb_varlen/sb_varlen_bwd.py:12-54).  Decides between that design and
// the two-pass backward of this library, which recomputes two score products instead.
//
// Each workgroup adds `reps` tiles of 32 x 128 floats into one of `ntiles` destination tiles
// (few tiles = heavy contention, many = none).  Two address patterns: the MFMA accumulator
// layout (a wave instruction touches 2 rows x 32 consecutive floats) and fully coalesced
// (64 consecutive floats).  Output: payload GB/s (4 bytes per atomic).
//
// Build and run:  make -C stickbreaking-attention_amd/csrc microbench && stickbreaking-attention_amd/lib/atomics
#include <hip/hip_runtime.h>

#include <cstdio>

template <bool COALESCED>
__global__ void __launch_bounds__(256) atomic_rate(float* buf, int ntiles, int reps) {
  const int w = threadIdx.x / 64, l = threadIdx.x % 64;
  for (int r = 0; r < reps; ++r) {
    const int tile = (blockIdx.x * 7 + r * 13) % ntiles;
    float* base = buf + (size_t)tile * 32 * 128;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      // accumulator layout: wave w owns columns 32w..32w+31; register i of lane (n, h) is row 8(i/4)+4h+i%4
      const int off = COALESCED ? (w * 16 + i) * 64 + l
                                : (8 * (i / 4) + 4 * (l / 32) + (i % 4)) * 128 + w * 32 + (l % 32);
      __builtin_amdgcn_global_atomic_fadd_f32((__attribute__((address_space(1))) float*)(base + off), 1.0f);
    }
  }
}

template <bool COALESCED>
static void run(int cus, int ntiles) {
  float* buf = nullptr;
  const size_t bytes = (size_t)ntiles * 32 * 128 * sizeof(float);
  if (hipMalloc(&buf, bytes) != hipSuccess) return;
  (void)hipMemset(buf, 0, bytes);
  const int reps = 64, blocks = cus * 4;
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  float ms = 0.f;
  for (int rep = 0; rep < 2; ++rep) {
    (void)hipEventRecord(e0);
    hipLaunchKernelGGL(atomic_rate<COALESCED>, dim3(blocks), dim3(256), 0, 0, buf, ntiles, reps);
    (void)hipEventRecord(e1);
    (void)hipEventSynchronize(e1);
    (void)hipEventElapsedTime(&ms, e0, e1);
  }
  const double payload = (double)blocks * reps * 32 * 128 * 4;
  std::printf("%-22s %6d destination tiles: %8.3f ms  %8.1f GB/s\n", COALESCED ? "coalesced" : "accumulator layout", ntiles, ms,
              payload / ms * 1e-6);
  std::fflush(stdout);
  (void)hipFree(buf);
}

int main() {
  int cus = 0;
  (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0);
  for (int ntiles : {64, 4096, 65536}) {
    run<false>(cus, ntiles);
    run<true>(cus, ntiles);
  }
  return 0;
}
