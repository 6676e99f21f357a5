// Entry point of the product family: checks the arguments and picks a kernel.
#include "gemm.h"

using namespace ninfer;

// force_generic != 0 runs the plain tiled kernel whatever the shape (tests
// compare the fast kernels with it).
extern "C" int ninfer_gemm(const GemmArgs* args, int force_generic, hipStream_t stream) {
  int rc = gemm_check(*args);
  if (rc) return rc;
  const GemmArgs& a = *args;
  if (!force_generic) {
    // many rows per weight matrix: 64-row tiles; few: 16-row tiles that stream the weights
    // (a product with few output features has too few 128-wide tiles to fill the GPU)
    bool many = a.offsets ? a.M >= 16 * a.groups : (a.M > 32 && a.N > 128);
    if (many && gemm_tile_takes(a)) return gemm_tile(a, stream);
    if (gemm_skinny_takes(a)) return gemm_skinny(a, stream);
  }
  return gemm_generic(a, stream);
}
