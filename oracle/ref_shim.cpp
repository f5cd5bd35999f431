// ref_shim.cpp -- extern "C" doors onto the reference's own SpMM-SpMM translation
// units, which are compiled where they lie in the reference checkout (see the
// Makefile; nothing of the reference is copied here).  TEST INFRASTRUCTURE ONLY:
// used to pin the C restatement in tf_oracle.c and, optionally, as the timed CPU
// baseline.  The product library never loads it.
//
// The declarations come from the reference's headers
// fusion/include/sparse-fusion/SpMM_SpMM.h and SpMM_SpMM_vectorized.h, found
// through the Makefile's -I flag.
#include "sparse-fusion/SpMM_SpMM.h"
#include "sparse-fusion/SpMM_SpMM_vectorized.h"

using namespace swiftware::sparse;

extern "C" {

// fusion/src/SpMM_SpMM.cpp:20-31
void ref_spmm_csr_sequential(int M, int N, int K, const int *Ap, const int *Ai,
                             const float *Ax, const float *Bx, float *Cx) {
  spmmCsrSequential<float>(M, N, K, Ap, Ai, Ax, Bx, Cx);
}

// fusion/src/SpMM_SpMM.cpp:37-55
void ref_spmm_csr_parallel(int M, int N, int K, const int *Ap, const int *Ai,
                           const float *Ax, const float *Bx, float *Cx, int NThreads) {
  spmmCsrParallel<float>(M, N, K, Ap, Ai, Ax, Bx, Cx, NThreads);
}

// fusion/src/SpMM_SpMM.cpp:211-248
void ref_spmm_spmm_fused_scalar(int M, int N, int K, int L, const int *Ap, const int *Ai,
                                const float *Ax, const int *Bp, const int *Bi,
                                const float *Bx, const float *Cx, float *Dx, float *ACx,
                                int LevelNo, const int *LevelPtr, const int *ParPtr,
                                const int *Partition, const int *ParType, int NThreads) {
  spmmCsrSpmmCsrFused<float>(M, N, K, L, Ap, Ai, Ax, Bp, Bi, Bx, Cx, Dx, ACx, LevelNo,
                             LevelPtr, ParPtr, Partition, ParType, NThreads);
}

// fusion/src/SpMM_SpMM_vectorized.cpp:876-989 (needs N % 32 == 0)
void ref_spmm_spmm_fused_vec32(int M, int N, int K, int L, const int *Ap, const int *Ai,
                               const float *Ax, const int *Bp, const int *Bi,
                               const float *Bx, const float *Cx, float *Dx, float *ACx,
                               int LevelNo, const int *LevelPtr, const int *ParPtr,
                               const int *Partition, const int *ParType, int NThreads) {
  spmmCsrSpmmCsrFusedVectorized2_32SP(M, N, K, L, Ap, Ai, Ax, Bp, Bi, Bx, Cx, Dx, ACx,
                                      LevelNo, LevelPtr, ParPtr, Partition, ParType,
                                      NThreads);
}

// fusion/src/SpMM_SpMM_vectorized.cpp:993-1110 (needs N % 32 == 0)
void ref_spmm_spmm_fused_separated_vec32(int M, int N, int K, int L, const int *Ap,
                                         const int *Ai, const float *Ax, const float *Cx,
                                         float *Dx, float *ACx, int LevelNo,
                                         const int *LevelPtr, const int *ParPtr,
                                         const int *Partition, const int *MixPtr,
                                         int NThreads) {
  spmmCsrSpmmCsrOneSparseMatrixFusedVectorized2_32SP(M, N, K, L, Ap, Ai, Ax, Cx, Dx, ACx,
                                                     LevelNo, LevelPtr, ParPtr, Partition,
                                                     MixPtr, NThreads);
}

// 1 when this CPU can run the build (the reference units are compiled with AVX-512 on).
int ref_cpu_ok(void) {
  return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma") &&
         __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512vl") &&
         __builtin_cpu_supports("avx512dq") && __builtin_cpu_supports("avx512bw");
}
}
