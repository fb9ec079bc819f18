// Microbenchmark behind the kernels' cost model: how far do matrix (MFMA) and vector (VALU) instructions of
// DIFFERENT wavefronts overlap on one SIMD of this GPU?  No memory traffic.  Three launches per row:
//   matrix alone   one workgroup of 4 wavefronts per CU (one wavefront per SIMD), all issuing independent MFMA
//   vector alone   the same, all issuing the vector mix
//   together       two workgroups per CU; on every SIMD one wavefront does the matrix work and one the vector work,
//                  each exactly what it did alone
// If the units overlapped, "together" would take max(matrix, vector); if they share the SIMD's time, the sum.
// Build: make -C long-context-modeling_amd/csrc ubench     Run: long-context-modeling_amd/lib/ubench_simd_overlap
#include <hip/hip_runtime.h>
#include <cstdio>
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
// MK: 0 = 32x32x16 C in VGPR, 1 = 32x32x16 C in AGPR, 2 = 16x16x32 (VGPR)
// VK: 0 = softmax mix (fma, exp, add, mul), 1 = fma only
// WHO: 0 = all waves MFMA, 1 = all waves VALU, 2 = even MFMA / odd VALU
template <int MK, int VK, int WHO>
__global__ void __launch_bounds__(256) k(int iters, float* out, float c) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(lane * 0.01f + i); b[i] = (__bf16)(lane * 0.02f - i); }
  f32x16 acc[4];
  f32x4 acc4[4];
  for (int j = 0; j < 4; ++j) { for (int r = 0; r < 16; ++r) acc[j][r] = 0.f; for (int r = 0; r < 4; ++r) acc4[j][r] = 0.f; }
  float v[32];
  for (int r = 0; r < 32; ++r) v[r] = lane * 0.001f + r;
  float sum = 0.f;
  const bool do_mfma = WHO == 0 || (WHO == 2 && ((wave + blockIdx.x) & 1) == 0);
  const bool do_valu = WHO == 1 || (WHO == 2 && ((wave + blockIdx.x) & 1) == 1);
  for (int it = 0; it < iters; ++it) {
    if (do_mfma) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (MK == 0) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j], 0, 0, 0);
          else if (MK == 1) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc[j]) : "v"(a), "v"(b));
          else { acc4[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc4[j], 0, 0, 0); acc4[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b, a, acc4[j], 0, 0, 0); }
        }
    }
    if (do_valu) {
#pragma unroll
      for (int r = 0; r < 32; ++r) {
        if (VK == 0) {
          const float e = __builtin_amdgcn_exp2f(fmaf(v[r], c, -1.0f));
          sum += e;
          v[r] = e * c;
        } else {
          v[r] = fmaf(v[r], c, 0.001f); v[r] = fmaf(v[r], c, 0.002f); v[r] = fmaf(v[r], c, 0.003f); v[r] = fmaf(v[r], c, 0.004f);
        }
      }
    }
  }
  float t = sum;
  for (int j = 0; j < 4; ++j) { for (int r = 0; r < 16; ++r) t += acc[j][r]; for (int r = 0; r < 4; ++r) t += acc4[j][r]; }
  for (int r = 0; r < 32; ++r) t += v[r];
  if (t == 12345.678f) out[0] = t;
}
template <int MK, int VK, int WHO> float run(int wgs_per_cu) {
  float* out; hipMalloc(&out, 4);
  const int iters = 2000, blocks = 256 * wgs_per_cu;
  hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
  hipLaunchKernelGGL((k<MK, VK, WHO>), dim3(blocks), dim3(256), 0, 0, iters, out, 0.999f);
  hipEventRecord(e0);
  hipLaunchKernelGGL((k<MK, VK, WHO>), dim3(blocks), dim3(256), 0, 0, iters, out, 0.999f);
  hipEventRecord(e1); hipEventSynchronize(e1);
  float ms; hipEventElapsedTime(&ms, e0, e1);
  hipFree(out);
  return ms;
}
template <int MK, int VK> void suite(const char* name) {
  // 2 WG/CU x 4 waves = 2 waves per SIMD; in WHO==2 one of them does MFMA and the other VALU, each doing what ONE wave does alone
  // compare: T(mfma alone, 1 wave/SIMD) , T(valu alone, 1 wave/SIMD), T(both, 2 waves/SIMD)
  const float tm = run<MK, VK, 0>(1), tv = run<MK, VK, 1>(1), tb = run<MK, VK, 2>(2);
  printf("%-44s mfma alone %.3f ms, valu alone %.3f ms, together %.3f ms  -> hidden fraction of the shorter: %.2f\n", name, tm, tv, tb,
         (tm + tv - tb) / (tm < tv ? tm : tv));
}
int main() {
  suite<0, 0>("32x32x16 C in VGPR  + softmax mix");
  suite<1, 0>("32x32x16 C in AGPR  + softmax mix");
  suite<2, 0>("16x16x32 (2 per slot) + softmax mix");
  suite<0, 1>("32x32x16 C in VGPR  + fma only");
  suite<1, 1>("32x32x16 C in AGPR  + fma only");
  suite<2, 1>("16x16x32 (2 per slot) + fma only");
  return 0;
}
