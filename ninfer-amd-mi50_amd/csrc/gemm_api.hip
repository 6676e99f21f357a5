// Entry point of the product family: checks the arguments and picks a kernel.
#include "gemm.h"
#include "moe_route.h"

using namespace ninfer;

// many rows per weight matrix: 64-row tiles and taller; few: 16-row tiles that stream the
// weights (a product with few output features has too few 128-wide tiles to fill the GPU).
// Grouped products count as many above 8 rows a group on average: some groups then have
// several 16-row tiles, each of which would stream the group's weights again (60 groups of
// 2 x 1408 x 2048 and 2048 x 1408: a 224-token portion 6.4 against 7.6 ms, 160 tokens 5.8
// against 6.4, the same at 8 and below; 64 groups of 2 x 2560 x 3584: 127 tokens 22.4 against 28.0,
// 80 tokens 21.7 against 23.1). A plain product of 17 to 32 rows whose weights are very large
// (256 Mi elements and more: a vocabulary's output head) counts as many too: the few-row
// kernel's second row tile would read them again, and they are beyond any cache (151,936 x
// 2048: 181 us there against 127 on the tile kernel; replayed decode steps of 17 to 32 rows
// 1% faster)
static bool many_rows(const GemmArgs& a) {
  if (a.offsets) return a.M > 8 * a.groups;
  const bool huge = a.M > 16 && a.epilogue == kEpilogueNone && (int64_t)a.N * a.K >= (256LL << 20);
  return (a.M > 32 || huge) && a.N > 128;
}

// force_generic != 0 runs the plain tiled kernel whatever the shape (tests
// compare the fast kernels with it).
extern "C" int ninfer_gemm(const GemmArgs* args, int force_generic, hipStream_t stream) {
  int rc = gemm_check(*args);
  if (rc) return rc;
  const GemmArgs& a = *args;
  if (!force_generic) {
    if (gemm_split_parts(a) >= 2) return gemm_split(a, stream);
    if (gemm_skinny_rows_takes(a)) return gemm_skinny_rows(a, stream);
    if (many_rows(a) && gemm_tile_takes(a)) return gemm_tile(a, stream);
    if (gemm_skinny_takes(a)) return gemm_skinny(a, stream);
  }
  return gemm_generic(a, stream);
}

// Into how many parts along K ninfer_gemm would cut this product (< 2: it would not).
extern "C" int ninfer_gemm_split_parts(const GemmArgs* args) {
  if (gemm_check(*args)) return 0;
  return gemm_split_parts(*args);
}

// Two products that do not depend on each other. Pairs of few-row products that have a
// kernel of their own run as one launch; all others one after the other.
extern "C" int ninfer_gemm_pair(const GemmArgs* a, const GemmArgs* b, int force_generic,
                                hipStream_t stream) {
  int rc = gemm_check(*a);
  if (rc) return rc;
  rc = gemm_check(*b);
  if (rc) return rc;
  if (!force_generic && !many_rows(*a) && !many_rows(*b) && gemm_skinny_pair_takes(*a, *b))
    return gemm_skinny_pair(*a, *b, stream);
  rc = ninfer_gemm(a, force_generic, stream);
  if (rc) return rc;
  return ninfer_gemm(b, force_generic, stream);
}

static int route_by(const GemmArgs& a, const RouteArgs& rt, hipStream_t stream) {
  const float* logits = (const float*)a.C;
  if (a.M <= 16) return ninfer_moe_route_small(logits, a.ldc, a.M, &rt, stream);
  if (rt.parts) return ninfer_moe_route_many(logits, a.ldc, a.M, &rt, stream);
  int rc = ninfer_router_topk(logits, a.ldc, a.M, &rt, stream);
  if (rc) return rc;
  return ninfer_moe_align(rt.ids, a.M * rt.k, rt.E, rt.offsets, rt.order, rt.tiles16,
                          rt.tiles_big, rt.tile_counts, stream);
}

static int route_check(const GemmArgs& a, const RouteArgs& rt) {
  NINFER_REQUIRE(!a.offsets && a.out_dtype == kF32 && a.N >= rt.E && a.ldc >= rt.E,
                 "gemm route: the product must be dense with 32-bit logits of %d experts", rt.E);
  NINFER_REQUIRE((!rt.tiles16) == (!rt.tiles_big) && (!rt.tiles16) == (!rt.tile_counts),
                 "gemm route: tile lists come together or not at all");
  NINFER_REQUIRE(rt.score == kScoreSoftmax || rt.score == kScoreSigmoid,
                 "gemm route: score function %d is neither softmax (0) nor sigmoid (1)", rt.score);
  NINFER_REQUIRE(route_groups_ok(rt), "gemm route: %d groups of which %d are open do not fit %d "
                 "experts and k=%d", rt.n_group, rt.topk_group, rt.E, rt.k);
  return 0;
}

// A router's logits (product `a`, [T, >= E] 32-bit: columns beyond the experts' are not the
// router's) and the routing of the rows by them. One launch where one block of the few-row
// kernel holds the product; otherwise the product, then the routing kernels.
extern "C" int ninfer_gemm_route(const GemmArgs* a, const RouteArgs* rt, int force_generic,
                                 hipStream_t stream) {
  int rc = gemm_check(*a);
  if (rc) return rc;
  rc = route_check(*a, *rt);
  if (rc) return rc;
  if (!force_generic && !many_rows(*a) && gemm_skinny_route_takes(*a, *rt))
    return gemm_skinny_route(*a, *rt, stream);
  rc = ninfer_gemm(a, force_generic, stream);
  if (rc) return rc;
  return route_by(*a, *rt, stream);
}

// The same with a second product `b` that does not depend on the first (a shared expert's gate
// and up) in the launch.
extern "C" int ninfer_gemm_pair_route(const GemmArgs* a, const GemmArgs* b, const RouteArgs* rt,
                                      int force_generic, hipStream_t stream) {
  int rc = gemm_check(*a);
  if (rc) return rc;
  rc = gemm_check(*b);
  if (rc) return rc;
  rc = route_check(*a, *rt);
  if (rc) return rc;
  if (!force_generic && !many_rows(*a) && !many_rows(*b) && gemm_skinny_route_pair_takes(*a, *b, *rt))
    return gemm_skinny_route_pair(*a, *b, *rt, stream);
  rc = ninfer_gemm_pair(a, b, force_generic, stream);
  if (rc) return rc;
  return route_by(*a, *rt, stream);
}
