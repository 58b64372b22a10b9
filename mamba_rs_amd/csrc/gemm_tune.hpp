// Choice of the vendor GEMM kernel for the projections that go to the library (prefill, and decode from 65-129 rows up; the reference sends them to cuBLAS with its default
// heuristics, src/mamba_ssm/gpu/blas.rs:771-811).  rocBLAS can list every kernel ("solution") able to run a problem; for
// the few shapes a prefill of given length uses, timing them once picks kernels 8-35 % faster than the default choice
// (measured: 16384 x 3072 x 768 60.7 -> 54.9 us, 16384 x 10240 x 2560 485 -> 432 us, 16384 x 192 x 5120 50 -> 32 us).
#pragma once
#include <hip/hip_runtime.h>

namespace mrs {

struct GemmTuner;
GemmTuner *gemm_tuner_create();
void gemm_tuner_destroy(GemmTuner *t);
void gemm_tuner_enable(GemmTuner *t, int on);
int gemm_tuner_enabled(const GemmTuner *t);

// C[m x n] = op(A) . B, column-major as rocBLAS sees them (alpha 1, beta 0, f32 accumulate); the types are rocblas_datatype
// values.  With tuning on, a problem of at least kTuneMinCols columns seen for the first time outside a stream capture
// is timed over all of the library's solutions (a few seconds; C is overwritten with the same product each time) and the
// fastest is used from then on; otherwise, and for every other call, the library's default choice runs.
constexpr int kTuneMinCols = 32;   // below that the engines run their own GEMM
int gemm_ex_tuned(GemmTuner *t, void *blas_handle, hipStream_t st, int trans_a, int m, int n, int k, const void *A, int a_type,
                  int lda, const void *B, int b_type, int ldb, void *C, int c_type, int ldc);

}  // namespace mrs
