// Launcher of the fp64 tile GEMM (gemm_f64.hip).
#ifndef VECOPS_HIP_GEMM_F64_H
#define VECOPS_HIP_GEMM_F64_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vecops_hip {

struct GemmF64Params {
  const double* a;    // [batch][M][K], element strides a_bs / a_rs / a_ks
  const double* b;    // [batch][N][K]
  const double* cin;  // null = none
  double* c;
  int32_t m, n, k, batch;
  int64_t a_rs, a_ks, a_bs;
  int64_t b_rs, b_ks, b_bs;
  int64_t c_rs, c_cs, c_bs;
  int64_t cin_rs, cin_cs, cin_bs;
};

// Enqueues C = C_in + A . B^T on `stream` (K = 0: C = C_in or zero).
hipError_t launch_gemm_f64(const GemmF64Params& p, hipStream_t stream);

}  // namespace vecops_hip
#endif
