// One epilogue kind of the INT8 GEMM family per translation unit: compiled once for every EpiKind value with
// -DTI_KIND=<n>, so that the kinds build in parallel.
#include "gemm_s8_impl.h"

#ifndef TI_KIND
#error "compile with -DTI_KIND=<EpiKind value>"
#endif
#define TI_CAT2(a, b) a##b
#define TI_CAT(a, b) TI_CAT2(a, b)

namespace ti {
int TI_CAT(launch_gemm_kind_, TI_KIND)(const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream) {
  return launch_kind<TI_KIND>(p, ws, ws_bytes, stream);
}
}  // namespace ti
