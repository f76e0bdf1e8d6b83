// How much ordinary VALU work hides under bf16 MFMAs on one gfx950 SIMD, and how fast a single
// wave can issue instructions: the two machine properties that bound the attention kernels
// of this library (each 32x32 score block costs 16-32 MFMAs AND 10-19 VALU instructions per
// score, so whether the two streams overlap decides the reachable fraction of the MFMA peak).
//
// Every kernel runs `reps` iterations of GROUPS groups; a group is one MFMA (or none) followed
// by VF independent fp32 FMAs and VT exp2 instructions, the order pinned with scheduling
// barriers.  One workgroup of 256 threads per CU and per occupancy step, so `waves/SIMD` is
// exact.  Output: nanoseconds of SIMD time per group.
//
// Build and run:  make -C stickbreaking-attention_amd/csrc microbench && stickbreaking-attention_amd/lib/coissue
#include <hip/hip_runtime.h>

#include <cstdio>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

template <int M, int VF, int VT>
__global__ void __launch_bounds__(256, 4) mix_kernel(float* out, int reps) {
  constexpr int GROUPS = 16;
  const int lane = threadIdx.x;
  bf16x8 a, b;
  for (int j = 0; j < 8; ++j) { a[j] = (__bf16)(0.01f * (lane + j)); b[j] = (__bf16)(0.02f * (lane - j)); }
  f32x16 acc[4];
  for (int i = 0; i < 4; ++i) for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
  float f[16], t[8];
  for (int j = 0; j < 16; ++j) f[j] = 0.001f * (lane + j);
  for (int j = 0; j < 8; ++j) t[j] = 0.001f * (lane + j);
#pragma unroll 1
  for (int r = 0; r < reps; ++r) {
#pragma unroll
    for (int m = 0; m < GROUPS; ++m) {
      if (M > 0) acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[m & 3], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int v = 0; v < VF; ++v) f[(v + m) & 15] = __builtin_fmaf(f[(v + m) & 15], 0.999f, 0.001f);
#pragma unroll
      for (int v = 0; v < VT; ++v) t[(v + m) & 7] = __builtin_amdgcn_exp2f(t[(v + m) & 7]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float sum = 0;
  for (int i = 0; i < 4; ++i) for (int j = 0; j < 16; ++j) sum += acc[i][j];
  for (int j = 0; j < 16; ++j) sum += f[j];
  for (int j = 0; j < 8; ++j) sum += t[j];
  out[blockIdx.x * 256 + threadIdx.x] = sum;
}

// Same question at a coarser grain: G MFMAs back to back (into four accumulators) followed by
// G * VF independent FMAs, 16 MFMAs per iteration.  Output: nanoseconds per MFMA (+ VF FMAs).
template <int G, int VF>
__global__ void __launch_bounds__(256, 4) grouped_kernel(float* out, int reps) {
  constexpr int TOTAL = 16;
  const int lane = threadIdx.x;
  bf16x8 a, b;
  for (int j = 0; j < 8; ++j) { a[j] = (__bf16)(0.01f * (lane + j)); b[j] = (__bf16)(0.02f * (lane - j)); }
  f32x16 acc[4];
  for (int i = 0; i < 4; ++i) for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
  float f[32];
  for (int j = 0; j < 32; ++j) f[j] = 0.001f * (lane + j);
#pragma unroll 1
  for (int r = 0; r < reps; ++r) {
#pragma unroll
    for (int g = 0; g < TOTAL / G; ++g) {
#pragma unroll
      for (int m = 0; m < G; ++m)
        acc[(g * G + m) & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[(g * G + m) & 3], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int v = 0; v < G * VF; ++v) f[(v + g) & 31] = __builtin_fmaf(f[(v + g) & 31], 0.999f, 0.001f);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float sum = 0;
  for (int i = 0; i < 4; ++i) for (int j = 0; j < 16; ++j) sum += acc[i][j];
  for (int j = 0; j < 32; ++j) sum += f[j];
  out[blockIdx.x * 256 + threadIdx.x] = sum;
}

template <int G, int VF>
static void run_grouped(float* out, int waves_per_simd) {
  const int reps = 20000;
  hipEvent_t e0, e1;
  hipEventCreate(&e0);
  hipEventCreate(&e1);
  int cus = 0;
  hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0);
  hipLaunchKernelGGL((grouped_kernel<G, VF>), dim3(cus * waves_per_simd), dim3(256), 0, 0, out, 10);
  hipDeviceSynchronize();
  hipEventRecord(e0);
  hipLaunchKernelGGL((grouped_kernel<G, VF>), dim3(cus * waves_per_simd), dim3(256), 0, 0, out, reps);
  hipEventRecord(e1);
  hipEventSynchronize(e1);
  float ms = 0.f;
  hipEventElapsedTime(&ms, e0, e1);
  std::printf("%d wave(s)/SIMD  %2d MFMA then %3d FMA               %6.2f ns per MFMA + %d FMA\n", waves_per_simd, G, G * VF,
              ms * 1e6 / reps / waves_per_simd / 16, VF);
  std::fflush(stdout);
}

template <int M, int VF, int VT>
static void run(float* out, int waves_per_simd, const char* what) {
  const int reps = 20000, groups = 16;
  hipEvent_t e0, e1;
  hipEventCreate(&e0);
  hipEventCreate(&e1);
  int cus = 0;
  hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0);
  hipLaunchKernelGGL((mix_kernel<M, VF, VT>), dim3(cus * waves_per_simd), dim3(256), 0, 0, out, 10);
  hipDeviceSynchronize();
  hipEventRecord(e0);
  hipLaunchKernelGGL((mix_kernel<M, VF, VT>), dim3(cus * waves_per_simd), dim3(256), 0, 0, out, reps);
  hipEventRecord(e1);
  hipEventSynchronize(e1);
  float ms = 0.f;
  hipEventElapsedTime(&ms, e0, e1);
  std::printf("%d wave(s)/SIMD  %-34s %6.2f ns per group\n", waves_per_simd, what, ms * 1e6 / reps / waves_per_simd / groups);
  std::fflush(stdout);
}

int main() {
  float* out = nullptr;
  if (hipMalloc(&out, 1024 * 4 * 256 * sizeof(float)) != hipSuccess) return 1;
  for (int w = 1; w <= 4; ++w) {
    run<1, 0, 0>(out, w, "1 MFMA 32x32x16 bf16");
    run<0, 8, 0>(out, w, "8 FMA");
    run<0, 0, 4>(out, w, "4 EXP2");
    run<1, 2, 0>(out, w, "1 MFMA + 2 FMA");
    run<1, 4, 0>(out, w, "1 MFMA + 4 FMA");
    run<1, 6, 0>(out, w, "1 MFMA + 6 FMA");
    run<1, 8, 0>(out, w, "1 MFMA + 8 FMA");
    run<1, 12, 0>(out, w, "1 MFMA + 12 FMA");
    run<1, 0, 2>(out, w, "1 MFMA + 2 EXP2");
    run<1, 0, 4>(out, w, "1 MFMA + 4 EXP2");
    run<1, 4, 2>(out, w, "1 MFMA + 4 FMA + 2 EXP2");
  }
  for (int w = 1; w <= 3; ++w) {
    run_grouped<1, 8>(out, w);
    run_grouped<4, 8>(out, w);
    run_grouped<16, 8>(out, w);
    run_grouped<1, 12>(out, w);
    run_grouped<16, 12>(out, w);
  }
  hipFree(out);
  return 0;
}
