// Host-side range check of the hash encoding's index arithmetic.
//
// The reference guards its lookups with tl.device_assert, active only under TRITON_DEBUG
// (triton_helpers/layers/hash_encoding/kernel.py:109-122, 151, 227-228).  Here the guard runs on the CPU: the very
// inline functions the kernels use (cell_index, rows_d3, rows_d2, corner_row; compiled with the same
// -ffp-contract=off) are evaluated for host coordinates, every corner row is compared with its level's size and the
// coordinates with [0, scale].  Nothing is launched; no GPU is needed.
#include <cmath>

#include "hash_common.h"

namespace nf {

template <int D>
static void check_points(const float* coords, int64_t n_points, const DevGeom& g, const int64_t* primes, float scale,
                         int variant, int64_t* rows_out, int64_t* n_bad_rows) {
  uint64_t pi64[D];
  uint32_t pi32[3] = {0u, 0u, 0u};
  for (int d = 0; d < D; ++d) {
    pi64[d] = (uint64_t)primes[d];
    if (d < 3) pi32[d] = (uint32_t)primes[d];
  }
  constexpr int CN = 1 << D;
  for (int64_t n = 0; n < n_points; ++n) {
    float x[D];
    for (int d = 0; d < D; ++d) {
      x[d] = coords[n * D + d];
      if (scale != 1.0f) x[d] = x[d] / scale;
    }
    for (int l = 0; l < g.levels; ++l) {
      const bool hashed = l >= g.first_hash;
      const uint32_t res = (uint32_t)g.res[l], n_rows = g.rows[l];
      uint64_t row[CN];
      if (variant == 1) {
        // the 32-bit form of the fast kernels: wrap-around products and a mask (D = 2, 3; power-of-two hashed levels)
        const Cell<D> cell = locate_cell<D>(x, g.res[l]);
        uint32_t c[3] = {cell.c[0], D > 1 ? cell.c[D > 1 ? 1 : 0] : 0u, D > 2 ? cell.c[D > 2 ? 2 : 0] : 0u};
        const Corner8 r = D == 3 ? rows_d3(c, hashed, res, n_rows - 1u, pi32) : rows_d2(c, hashed, res, n_rows - 1u, pi32);
        for (int j = 0; j < CN; ++j) row[j] = r.row[j];
      } else {
        const Cell<D> cell = locate_cell<D>(x, g.res[l]);
        for (int j = 0; j < CN; ++j) row[j] = corner_row<D>(cell, j, hashed, res, n_rows, pi64);
      }
      for (int j = 0; j < CN; ++j) {
        if (row[j] >= (uint64_t)n_rows) ++*n_bad_rows;
        if (rows_out != nullptr) rows_out[(n * g.levels + l) * CN + j] = (int64_t)row[j];
      }
    }
  }
}

}  // namespace nf

using namespace nf;

extern "C" int nf_hash_check_host(const float* coords, int64_t n_points, const nf_hash_geom* geom, const int64_t* primes,
                                  float scale, int variant, int64_t* rows_out, int64_t* n_bad_rows, int64_t* n_bad_coords) {
  DevGeom g;
  if (int rc = make_dev_geom(geom, &g)) return rc;
  NF_REQUIRE(n_points >= 0, NF_EINVAL, "n_points negative");
  NF_REQUIRE(scale > 0.0f, NF_EINVAL, "scale must be positive");
  NF_REQUIRE(variant == 0 || variant == 1, NF_EINVAL, "variant=%d must be 0 (64-bit) or 1 (32-bit)", variant);
  NF_REQUIRE(n_bad_rows != nullptr && n_bad_coords != nullptr, NF_EINVAL, "NULL counter argument");
  *n_bad_rows = 0;
  *n_bad_coords = 0;
  if (n_points == 0) return 0;
  NF_REQUIRE(coords && primes, NF_EINVAL, "NULL pointer argument");
  if (variant == 1) {
    NF_REQUIRE(g.dims == 2 || g.dims == 3, NF_EUNSUPPORTED, "the 32-bit index form covers 2 and 3 dimensions, got %d", g.dims);
    for (int l = g.first_hash < 0 ? 0 : g.first_hash; l < g.levels; ++l)
      NF_REQUIRE((g.rows[l] & (g.rows[l] - 1u)) == 0u, NF_EUNSUPPORTED,
                 "the 32-bit index form needs power-of-two hashed levels (level %d has %u rows)", l, g.rows[l]);
  }
  for (int64_t i = 0; i < n_points * g.dims; ++i) {
    const float v = coords[i];
    if (!(v >= 0.0f && v <= scale)) ++*n_bad_coords;  // NaN fails both comparisons
  }
  switch (g.dims) {
    case 1: check_points<1>(coords, n_points, g, primes, scale, variant, rows_out, n_bad_rows); break;
    case 2: check_points<2>(coords, n_points, g, primes, scale, variant, rows_out, n_bad_rows); break;
    case 3: check_points<3>(coords, n_points, g, primes, scale, variant, rows_out, n_bad_rows); break;
    case 4: check_points<4>(coords, n_points, g, primes, scale, variant, rows_out, n_bad_rows); break;
    case 5: check_points<5>(coords, n_points, g, primes, scale, variant, rows_out, n_bad_rows); break;
    default: check_points<6>(coords, n_points, g, primes, scale, variant, rows_out, n_bad_rows); break;
  }
  return 0;
}
