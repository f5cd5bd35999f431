// Measurement aid: do fp32 MFMA instructions and fp32 VALU instructions of different wavefronts overlap on a SIMD?
// The fused GeMM-SpMM kernels run a wavefront that computes the intermediate on the MFMA path beside one that
// gathers and multiplies on the VALU on every SIMD; what the pair can reach depends on whether the two kinds of
// instruction share the SIMD's issue.  One workgroup of 512 threads per compute unit: wavefronts w and w + 4 share
// SIMD w.  Every wavefront runs `iters` rounds of 32 independent-enough instructions of its kind:
//   MFMA: 32 x v_mfma_f32_16x16x4_f32 (or 32 x v_mfma_f32_16x16x32_bf16) on four accumulators in turn
//   FMA : 256 x v_fma_f32 on eight accumulators in turn
#include <hip/hip_runtime.h>

#include "tf_internal.h"

namespace tf {

typedef float cal_v4f __attribute__((ext_vector_type(4)));
typedef short cal_v8s __attribute__((ext_vector_type(8)));

enum { kCalNone = 0, kCalMfmaF32 = 1, kCalFma = 2, kCalMfmaBf16 = 3 };

// role_lo: what wavefronts 0-3 (the older one of every SIMD) do, role_hi: wavefronts 4-7.
__global__ __launch_bounds__(512) void issue_probe_kernel(float *__restrict__ out, int iters, int role_lo, int role_hi) {
  const int role = threadIdx.x < 256 ? role_lo : role_hi;
  float r = 0.f;
  if (role == kCalMfmaF32) {
    cal_v4f acc[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    const float a = threadIdx.x * 1e-3f, b = 1.0f + threadIdx.x * 1e-4f;
    for (int i = 0; i < iters; ++i) {
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[j], 0, 0, 0);
    }
    r = acc[0][0] + acc[1][1] + acc[2][2] + acc[3][3];
  } else if (role == kCalMfmaBf16) {
    cal_v4f acc[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    cal_v8s a, b;
    for (int j = 0; j < 8; ++j) { a[j] = (short)(threadIdx.x + j); b[j] = (short)(threadIdx.x * 3 + j); }
    for (int i = 0; i < iters; ++i) {
#pragma unroll
      for (int u = 0; u < 8; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[j], 0, 0, 0);
    }
    r = acc[0][0] + acc[1][1] + acc[2][2] + acc[3][3];
  } else if (role == kCalFma) {
    float x[8];
    for (int j = 0; j < 8; ++j) x[j] = threadIdx.x * 1e-3f + j;
    const float m = 1.0f + threadIdx.x * 1e-7f, c = 1e-3f;
    for (int i = 0; i < iters; ++i) {
#pragma unroll
      for (int u = 0; u < 32; ++u)
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = __builtin_fmaf(x[j], m, c);
    }
    for (int j = 0; j < 8; ++j) r += x[j];
  }
  if (r == 123.456f) out[threadIdx.x] = r;  // (keeps the loops)
}

hipError_t launch_issue_probe(float *out, int compute_units, int iters, int role_lo, int role_hi, hipStream_t st) {
  hipLaunchKernelGGL(issue_probe_kernel, dim3(compute_units), dim3(512), 0, st, out, iters, role_lo, role_hi);
  return hipGetLastError();
}

}  // namespace tf
