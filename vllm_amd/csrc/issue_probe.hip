// Measurement probe (not part of the GEMM library): how the matrix pipe and the vector ALU of a gfx950 SIMD share
// issue time.  Each wavefront runs a loop of independent in-place MFMAs (v_mfma_f32_16x16x32_f16 on 32 different
// accumulators) with NV other VALU instructions after each MFMA, either independent of each other (eight registers used
// in turn) or one dependent chain.  Timed with events around the launch; one workgroup per compute unit, 4 or 8
// wavefronts per workgroup (one or two per SIMD).  Built into its own small library and only called by
// `bench.py --issue-probe`.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int NV, bool DEP>
__global__ __launch_bounds__(512) void issue_probe_kernel(const uint32_t* __restrict__ in, float* __restrict__ out, int iters) {
  f32x4 acc[32];
#pragma unroll
  for (int i = 0; i < 32; ++i) acc[i] = f32x4{0, 0, 0, 0};
  const int t = threadIdx.x;
  u32x4 a[4], b[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = *(const u32x4*)(in + ((t * 6 + i) * 4) % 4096);
#pragma unroll
  for (int i = 0; i < 2; ++i) b[i] = *(const u32x4*)(in + ((t * 6 + 4 + i) * 4) % 4096);
  uint32_t v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = in[(t + 11 * i) % 4096];
  uint32_t mask = 0x000f000fu, ex = 0x64006400u;
  asm volatile("" : "+v"(mask), "+v"(ex));
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a[i >> 3]), "v"(b[i & 1]));
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        if (DEP)
          asm volatile("v_and_or_b32 %0, %0, %1, %2" : "+v"(v[0]) : "v"(mask), "v"(ex));
        else
          asm volatile("v_and_or_b32 %0, %0, %1, %2" : "+v"(v[(i * NV + j) & 7]) : "v"(mask), "v"(ex));
      }
    }
  }
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  float s = 0;
#pragma unroll
  for (int i = 0; i < 32; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  uint32_t x = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) x ^= v[i];
  out[(size_t)blockIdx.x * blockDim.x + t] = s + (float)x;
}

typedef void (*probe_fn)(const uint32_t*, float*, int);
template <bool DEP>
static probe_fn pick(int nv) {
  switch (nv) {
    case 0: return issue_probe_kernel<0, DEP>;
    case 1: return issue_probe_kernel<1, DEP>;
    case 2: return issue_probe_kernel<2, DEP>;
    case 3: return issue_probe_kernel<3, DEP>;
    case 4: return issue_probe_kernel<4, DEP>;
    case 5: return issue_probe_kernel<5, DEP>;
    case 6: return issue_probe_kernel<6, DEP>;
    default: return nullptr;
  }
}

// in: 4096 dwords of operand data on the device; out: >= workgroups * 512 floats.  Returns the best of three timed
// launches in milliseconds (negative on error).  MFMAs per wavefront = iters * 32.
extern "C" float w4a16_issue_probe(const uint32_t* in, float* out, int workgroups, int waves_per_wg, int nv, int dependent,
                                   int iters) {
  probe_fn fn = dependent ? pick<true>(nv) : pick<false>(nv);
  if (!fn || (waves_per_wg != 4 && waves_per_wg != 8) || workgroups <= 0) return -1.0f;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -2.0f;
  hipLaunchKernelGGL(fn, dim3(workgroups), dim3(waves_per_wg * 64), 0, 0, in, out, 20);
  if (hipDeviceSynchronize() != hipSuccess) return -3.0f;
  float best = 1e30f;
  for (int rep = 0; rep < 3; ++rep) {
    hipEventRecord(e0, 0);
    hipLaunchKernelGGL(fn, dim3(workgroups), dim3(waves_per_wg * 64), 0, 0, in, out, iters);
    hipEventRecord(e1, 0);
    if (hipEventSynchronize(e1) != hipSuccess) return -4.0f;
    float ms = 0;
    hipEventElapsedTime(&ms, e0, e1);
    if (ms < best) best = ms;
  }
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  return best;
}
