// Pieces shared by the hash-encoding translation units (compiled with -ffp-contract=off).
#pragma once

#include "nf_common.h"

namespace nf {

struct DevGeom {
  int dims, feat, levels, first_hash;
  uint64_t max_rows;
  int res[NF_MAX_LEVELS];
  uint32_t rows[NF_MAX_LEVELS];
  int64_t row_offset[NF_MAX_LEVELS];
};


constexpr int TILE_THREADS = 256;

struct Corner8 {
  uint32_t row[8];
};

// Cell of a scaled coordinate: floor(pos) kept inside [0, res].  Coordinates in [0, scale] are unaffected (their
// floor is already there); anything else -- slightly negative from normalisation noise, beyond scale, inf, NaN --
// lands on an edge cell instead of indexing outside the level (fmaxf(NaN, 0) is 0).  The reference only asserts the
// range in its debug build (triton_helpers/layers/hash_encoding/kernel.py:227-228).
__host__ __device__ __forceinline__ uint32_t cell_index(float fl, float fres) {
  return (uint32_t)(int)fminf(fmaxf(fl, 0.0f), fres);
}

__host__ __device__ __forceinline__ Corner8 rows_d3(const uint32_t c[3], bool hashed, uint32_t res, uint32_t mask,
                                           const uint32_t pi[3]) {
  Corner8 r;
  if (hashed) {
    // (c+1)*pi == c*pi + pi in 32-bit wrap-around arithmetic; the low 32 bits of the
    // 64-bit products are all a power-of-two modulus keeps.
    const uint32_t x0 = c[0] * pi[0], x1 = x0 + pi[0];
    const uint32_t y0 = c[1] * pi[1], y1 = y0 + pi[1];
    const uint32_t z0 = c[2] * pi[2], z1 = z0 + pi[2];
    r.row[0] = (x0 ^ y0 ^ z0) & mask;
    r.row[1] = (x1 ^ y0 ^ z0) & mask;
    r.row[2] = (x0 ^ y1 ^ z0) & mask;
    r.row[3] = (x1 ^ y1 ^ z0) & mask;
    r.row[4] = (x0 ^ y0 ^ z1) & mask;
    r.row[5] = (x1 ^ y0 ^ z1) & mask;
    r.row[6] = (x0 ^ y1 ^ z1) & mask;
    r.row[7] = (x1 ^ y1 ^ z1) & mask;
  } else {
    const uint32_t r2 = res * res;
    const uint32_t b = c[0] + c[1] * res + c[2] * r2;
    r.row[0] = b;
    r.row[1] = b + 1;
    r.row[2] = b + res;
    r.row[3] = b + res + 1;
    r.row[4] = b + r2;
    r.row[5] = b + r2 + 1;
    r.row[6] = b + r2 + res;
    r.row[7] = b + r2 + res + 1;
  }
  return r;
}

// The same for two dimensions (rows 0..3 of the result are used).
__host__ __device__ __forceinline__ Corner8 rows_d2(const uint32_t c[3], bool hashed, uint32_t res, uint32_t mask, const uint32_t pi[3]) {
  Corner8 r;
  if (hashed) {
    const uint32_t x0 = c[0] * pi[0], x1 = x0 + pi[0];
    const uint32_t y0 = c[1] * pi[1], y1 = y0 + pi[1];
    r.row[0] = (x0 ^ y0) & mask;
    r.row[1] = (x1 ^ y0) & mask;
    r.row[2] = (x0 ^ y1) & mask;
    r.row[3] = (x1 ^ y1) & mask;
  } else {
    // x == scale in both dimensions puts the last corner (weight 0) at row (res+1)^2, one past the level: keep it inside
    const uint32_t b = c[0] + c[1] * res;
    r.row[0] = b;
    r.row[1] = b + 1;
    r.row[2] = b + res;
    r.row[3] = b + res + 1 < mask ? b + res + 1 : mask;
  }
  r.row[4] = r.row[5] = r.row[6] = r.row[7] = 0u;
  return r;
}

__host__ __device__ __forceinline__ void weights_d2(const float f[3], float w[8]) {
  const float gx = 1.0f - f[0], gy = 1.0f - f[1];
  w[0] = gx * gy;
  w[1] = f[0] * gy;
  w[2] = gx * f[1];
  w[3] = f[0] * f[1];
}

__host__ __device__ __forceinline__ void weights_d3(const float f[3], float w[8]) {
  const float gx = 1.0f - f[0], gy = 1.0f - f[1], gz = 1.0f - f[2];
  w[0] = (gx * gy) * gz;
  w[1] = (f[0] * gy) * gz;
  w[2] = (gx * f[1]) * gz;
  w[3] = (f[0] * f[1]) * gz;
  w[4] = (gx * gy) * f[2];
  w[5] = (f[0] * gy) * f[2];
  w[6] = (gx * f[1]) * f[2];
  w[7] = (f[0] * f[1]) * f[2];
}

// ---- generic form: any D <= NF_MAX_DIMS, any level size (exact 64-bit remainder) ----
template <int D>
struct Cell {
  uint32_t c[D];
  float frac[D];
};

// x: the point's coordinates already divided by scale
template <int D>
__host__ __device__ __forceinline__ Cell<D> locate_cell(const float* x, int res) {
  Cell<D> r;
  const float fres = (float)res;
#pragma unroll
  for (int d = 0; d < D; ++d) {
    const float pos = x[d] * fres;
    const float fl = floorf(pos);
    r.c[d] = cell_index(fl, fres);
    r.frac[d] = pos - fl;
  }
  return r;
}

template <int D>
__host__ __device__ __forceinline__ uint64_t corner_row(const Cell<D>& cell, int j, bool hashed, uint32_t res, uint32_t rows,
                                                        const uint64_t* pi) {
  if (!hashed) {
    uint64_t idx = 0, stride = 1;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      idx += (uint64_t)(cell.c[d] + ((j >> d) & 1)) * stride;
      stride *= res;
    }
    // D <= 2: the last corner of x == scale (weight 0) would be row (res+1)^D, one past the level
    return D <= 2 && idx >= rows ? (uint64_t)rows - 1 : idx;
  }
  uint64_t h = 0;
#pragma unroll
  for (int d = 0; d < D; ++d) h ^= (uint64_t)(cell.c[d] + ((j >> d) & 1)) * pi[d];
  // power-of-two sizes take the mask; anything else the exact 64-bit remainder
  return (rows & (rows - 1)) == 0 ? (h & (uint64_t)(rows - 1)) : (h % (uint64_t)rows);
}

template <int D>
__host__ __device__ __forceinline__ float corner_weight(const Cell<D>& cell, int j) {
  float w = ((j & 1) ? cell.frac[0] : 1.0f - cell.frac[0]);
#pragma unroll
  for (int d = 1; d < D; ++d) w = w * (((j >> d) & 1) ? cell.frac[d] : 1.0f - cell.frac[d]);
  return w;
}

inline int make_dev_geom(const nf_hash_geom* geom, DevGeom* d) {
  NF_REQUIRE(geom != nullptr, NF_EINVAL, "geom is NULL");
  NF_REQUIRE(geom->dims >= 1 && geom->dims <= NF_MAX_DIMS, NF_EINVAL, "dims=%d outside 1..%d", geom->dims,
             NF_MAX_DIMS);
  NF_REQUIRE(geom->feat >= 1, NF_EINVAL, "feat=%d must be positive", geom->feat);
  NF_REQUIRE(geom->levels >= 1 && geom->levels <= NF_MAX_LEVELS, NF_EINVAL, "levels=%d outside 1..%d", geom->levels,
             NF_MAX_LEVELS);
  d->dims = geom->dims;
  d->feat = geom->feat;
  d->levels = geom->levels;
  d->first_hash = geom->first_hash_level;
  d->max_rows = (uint64_t)geom->max_rows;
  for (int l = 0; l < geom->levels; ++l) {
    NF_REQUIRE(geom->res[l] >= 1, NF_EINVAL, "res[%d]=%d must be positive", l, geom->res[l]);
    NF_REQUIRE(geom->rows[l] >= 1 && geom->rows[l] < (int64_t)1 << 32, NF_EINVAL, "rows[%d]=%lld outside 1..2^32-1", l,
               (long long)geom->rows[l]);
    NF_REQUIRE(geom->row_offset[l] >= 0, NF_EINVAL, "row_offset[%d] negative", l);
    // a dense level must be able to hold every corner the stride-N_l indexing can produce
    if (l < geom->first_hash_level) {
      double need = 1.0;
      for (int k = 0; k < geom->dims; ++k) need *= (double)geom->res[l] + 1.0;
      NF_REQUIRE(need <= (double)geom->rows[l], NF_EINVAL, "level %d marked dense but (res+1)^D > rows", l);
    }
    d->res[l] = geom->res[l];
    d->rows[l] = (uint32_t)geom->rows[l];
    d->row_offset[l] = geom->row_offset[l];
  }
  return 0;
}


// backward through LDS tiles (hash_encoding_bwd_scan.hip)
int64_t bwd_scan_workspace_bytes(int64_t n_points, const nf_hash_geom* geom, int dout_dtype);
int launch_bwd_scan(const void* coords, int cdt, int64_t csn, int64_t csd, const void* dout, int ddt, int64_t dout_stride,
                    float* dtable, int64_t N, const nf_hash_geom* geom, const DevGeom& g, const int64_t* primes, float scale,
                    void* workspace, hipStream_t s);


// backward by binning the contributions per table stretch (hash_encoding_bwd_bin.hip)
int64_t bwd_bin_workspace_bytes(int64_t n_points, const nf_hash_geom* geom, int dout_dtype, int flags);
// whether launch_bwd_bin would walk the points without records (small tables; also for batches too small for the records)
bool bwd_direct_applies(int64_t n_points, const nf_hash_geom* geom, int flags);
int launch_bwd_bin(const void* coords, int cdt, int64_t csn, int64_t csd, const void* dout, int ddt, int64_t dout_stride,
                   float* dtable, int64_t N, const nf_hash_geom* geom, const DevGeom& g, const int64_t* primes, float scale,
                   void* workspace, int flags, hipStream_t s);

}  // namespace nf
