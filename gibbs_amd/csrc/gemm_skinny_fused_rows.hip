// The fused few-row products (gemm_skinny_fused.hip) for a row-major W: a translation unit of its own, so that the
// two sets of instantiations compile side by side.
#include "gemm_skinny_fused.h"

// args: a FusedArgs that an entry point of gemm_skinny_fused.hip has filled in and checked; epilogue: its EPI_ code.
void gibbs_fused_rows(const void* args, int epilogue, int rms, hipStream_t stream) {
  const FusedArgs& a = *(const FusedArgs*)args;
  switch (epilogue) {
    case EPI_STORE: run_store<false>(a, rms != 0, stream); break;
    case EPI_RESIDUAL: run_residual<false>(a, stream); break;
    case EPI_GLU: run_glu<false>(a, rms != 0, stream); break;
    default: run_conv<false>(a, rms != 0, stream); break;
  }
}
