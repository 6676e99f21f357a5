// Entry point of the product family: checks the arguments and picks a kernel.
#include "gemm.h"

using namespace ninfer;

// force_generic != 0 runs the plain tiled kernel whatever the shape (tests
// compare the fast kernels with it).
extern "C" int ninfer_gemm(const GemmArgs* args, int force_generic, hipStream_t stream) {
  int rc = gemm_check(*args);
  if (rc) return rc;
  (void)force_generic;
  return gemm_generic(*args, stream);
}
