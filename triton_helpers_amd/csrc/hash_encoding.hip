// Multiresolution hash encoding for gfx950: forward gather, backward scatter-add,
// and an index/weight dump used for bit-exact index checks.
//
// Arithmetic contract (follows the PyTorch path of the reference,
// triton_helpers/layers/hash_encoding/kernel.py:448-479):
//   pos   = fp32(x / scale) * fp32(N_l)          one rounding per operation, no FMA
//   cell  = floor(pos),  frac = pos - floor(pos)
//   dense level  ((N_l+1)^D <= T):  row = sum_d (cell_d + bit_d) * N_l^d
//   hashed level:                   row = (xor_d (cell_d + bit_d) * pi_d) mod T_l   (64-bit products)
//   weight_j = prod_d (bit_d ? frac_d : 1 - frac_d),   out = sum_j weight_j * table[row_j]
// The file is compiled with -ffp-contract=off so that none of this is fused.
#include "hash_common.h"

namespace nf {

// ---------------------------------------------------------------------------
// Generic path: one thread per (point, level); any D <= 4, any F, any dtype mix.
// ---------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ Cell<D> locate(const void* coords, int cdt, int64_t sn, int64_t sd, int64_t n, float scale,
                                          int res) {
  float x[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    x[d] = load_as_f32(coords, n * sn + d * sd, cdt);
    if (scale != 1.0f) x[d] = x[d] / scale;
  }
  return locate_cell<D>(x, res);
}

template <int D>
__device__ __forceinline__ void load_primes(const int64_t* primes, uint64_t* pi) {
#pragma unroll
  for (int d = 0; d < D; ++d) pi[d] = (uint64_t)primes[d];
}

// V = features per load: rows whose width, base and output allow it are read V features (4, 8 or 16 bytes) at a time,
// every feature summed over the corners in the same order as with V = 1
template <int D, typename TT, int V = 1>
__global__ __launch_bounds__(256) void hash_fwd_generic_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                          const typename TT::storage* table,
                                                          typename TT::storage* out, int64_t out_stride, int64_t N,
                                                          DevGeom g, const int64_t* primes, float scale) {
  typedef typename TT::storage S;
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int l = blockIdx.y;
  if (n >= N) return;
  uint64_t pi[D];
  load_primes<D>(primes, pi);
  const bool hashed = l >= g.first_hash;
  const Cell<D> cell = locate<D>(coords, cdt, csn, csd, n, scale, g.res[l]);
  const S* tab = table + g.row_offset[l] * g.feat;
  uint64_t rows[1 << D];
  float w[1 << D];
#pragma unroll
  for (int j = 0; j < (1 << D); ++j) {
    rows[j] = corner_row<D>(cell, j, hashed, (uint32_t)g.res[l], g.rows[l], pi);
    w[j] = corner_weight<D>(cell, j);
  }
  if constexpr (V == 1) {
    for (int f = 0; f < g.feat; ++f) {
      float acc = 0.0f;
#pragma unroll
      for (int j = 0; j < (1 << D); ++j) acc = acc + w[j] * TT::to_f32(tab[rows[j] * g.feat + f]);
      out[n * out_stride + (int64_t)l * g.feat + f] = TT::from_f32(acc);
    }
  } else {
    struct alignas(V * sizeof(S)) Piece { S v[V]; };
    for (int f = 0; f < g.feat; f += V) {
      float acc[V];
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = 0.0f;
      Piece q[1 << D];
#pragma unroll
      for (int j = 0; j < (1 << D); ++j) q[j] = *reinterpret_cast<const Piece*>(tab + rows[j] * g.feat + f);
#pragma unroll
      for (int j = 0; j < (1 << D); ++j)
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] = acc[e] + w[j] * TT::to_f32(q[j].v[e]);
      Piece r;
#pragma unroll
      for (int e = 0; e < V; ++e) r.v[e] = TT::from_f32(acc[e]);
      *reinterpret_cast<Piece*>(out + n * out_stride + (int64_t)l * g.feat + f) = r;
    }
  }
}

template <int D>
__global__ __launch_bounds__(256) void hash_bwd_generic_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                          const void* dout, int ddt, int64_t dout_stride,
                                                          float* dtable, int64_t N, DevGeom g, const int64_t* primes,
                                                          float scale) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int l = blockIdx.y;
  if (n >= N) return;
  uint64_t pi[D];
  load_primes<D>(primes, pi);
  const bool hashed = l >= g.first_hash;
  const Cell<D> cell = locate<D>(coords, cdt, csn, csd, n, scale, g.res[l]);
  float* tab = dtable + g.row_offset[l] * g.feat;
  for (int f = 0; f < g.feat; ++f) {
    const float go = load_as_f32(dout, n * dout_stride + (int64_t)l * g.feat + f, ddt);
#pragma unroll
    for (int j = 0; j < (1 << D); ++j) {
      const uint64_t row = corner_row<D>(cell, j, hashed, (uint32_t)g.res[l], g.rows[l], pi);
      unsafeAtomicAdd(tab + row * g.feat + f, corner_weight<D>(cell, j) * go);
    }
  }
}

template <int D>
__global__ __launch_bounds__(256) void hash_indices_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                      int64_t* out_rows, float* out_w, int64_t N, DevGeom g,
                                                      const int64_t* primes, float scale) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int l = blockIdx.y;
  if (n >= N) return;
  uint64_t pi[D];
  load_primes<D>(primes, pi);
  const bool hashed = l >= g.first_hash;
  const Cell<D> cell = locate<D>(coords, cdt, csn, csd, n, scale, g.res[l]);
  const int64_t base = (n * g.levels + l) * (1 << D);
#pragma unroll
  for (int j = 0; j < (1 << D); ++j) {
    out_rows[base + j] = (int64_t)corner_row<D>(cell, j, hashed, (uint32_t)g.res[l], g.rows[l], pi);
    if (out_w) out_w[base + j] = corner_weight<D>(cell, j);
  }
}

// The same table through the index arithmetic of the fast kernels (sweep, tiled, binned backward): cells from
// cell_index(), rows from rows_d3() / rows_d2() in 32-bit wrap-around arithmetic with the level's mask, weights from
// weights_d3() / weights_d2() -- the very inline functions those kernels call, here with their results written out.
template <int D>
__global__ __launch_bounds__(256) void hash_indices_fast_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                           int64_t* out_rows, float* out_w, int64_t N, DevGeom g,
                                                           const int64_t* primes, float scale) {
  static_assert(D == 2 || D == 3, "the fast kernels cover two and three dimensions");
  constexpr int CN = 1 << D;
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int l = blockIdx.y;
  if (n >= N) return;
  uint32_t pi[3] = {0u, 0u, 0u};
#pragma unroll
  for (int d = 0; d < D; ++d) pi[d] = (uint32_t)primes[d];
  float x[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int d = 0; d < D; ++d) {
    x[d] = load_as_f32(coords, n * csn + d * csd, cdt);
    if (scale != 1.0f) x[d] = x[d] / scale;
  }
  const bool hashed = l >= g.first_hash;
  const uint32_t res = (uint32_t)g.res[l];
  const float fres = (float)g.res[l];
  const uint32_t mask = g.rows[l] - 1;
  uint32_t c[3] = {0u, 0u, 0u};
  float fr[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int d = 0; d < D; ++d) {
    const float pos = x[d] * fres;
    const float fl = floorf(pos);
    c[d] = cell_index(fl, fres);
    fr[d] = pos - fl;
  }
  const Corner8 r = D == 3 ? rows_d3(c, hashed, res, mask, pi) : rows_d2(c, hashed, res, mask, pi);
  float w[8];
  if (D == 3) weights_d3(fr, w);
  else weights_d2(fr, w);
  const int64_t base = (n * g.levels + l) * CN;
#pragma unroll
  for (int j = 0; j < CN; ++j) {
    out_rows[base + j] = (int64_t)r.row[j];
    if (out_w) out_w[base + j] = w[j];
  }
}

// ---------------------------------------------------------------------------
// Tiled path: D = 3, F = 2, 16-bit tables (one table row = one dword), L % 4 == 0.
//
// A workgroup of 256 threads owns P = 256*PPT consecutive points and walks the
// levels in order, so that the workgroups resident on an XCD touch the same
// one or two level tables at a time and those stay in that XCD's L2.  Results
// are staged in LDS as stage[level][point] (row stride P+2 dwords) and leave
// as full 16-byte pieces of contiguous output rows; the backward stages the
// incoming gradient rows the same way before scattering.
// ---------------------------------------------------------------------------
// FW: 32-bit words (feature pairs) per table row; a corner's FW words share a cache line, so the pairs after the
// first cost no further line fetch.
template <typename TT, int PPT, int FW>
__global__ __launch_bounds__(TILE_THREADS) void hash_fwd_tiled_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                                 const uint32_t* table, uint16_t* out,
                                                                 int64_t out_stride, int64_t N, DevGeom g,
                                                                 const int64_t* primes, float scale) {
  constexpr int P = TILE_THREADS * PPT;
  constexpr int LD = P + 2;
  extern __shared__ uint32_t stage[];
  const int t = threadIdx.x;
  const int64_t p0 = (int64_t)blockIdx.x * P;
  const int L = g.levels;

  float x[PPT][3];
#pragma unroll
  for (int i = 0; i < PPT; ++i) {
    int64_t n = p0 + t + TILE_THREADS * i;
    if (n >= N) n = N - 1;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
      float v = load_as_f32(coords, n * csn + d * csd, cdt);
      x[i][d] = scale != 1.0f ? v / scale : v;
    }
  }
  const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], (uint32_t)primes[2]};

  for (int l = 0; l < L; ++l) {
    const uint32_t res = (uint32_t)g.res[l];
    const float fres = (float)g.res[l];
    const bool hashed = l >= g.first_hash;
    const uint32_t mask = g.rows[l] - 1;
    const uint32_t* tab = table + g.row_offset[l] * FW;
    uint32_t v[PPT][8][FW];
    float w[PPT][8];
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      uint32_t c[3];
      float fr[3];
#pragma unroll
      for (int d = 0; d < 3; ++d) {
        const float pos = x[i][d] * fres;
        const float fl = floorf(pos);
        c[d] = cell_index(fl, fres);
        fr[d] = pos - fl;
      }
      const Corner8 r = rows_d3(c, hashed, res, mask, pi);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (FW == 1) {
          v[i][j][0] = tab[r.row[j]];
        } else if (FW == 2) {
          const uint2 q = *reinterpret_cast<const uint2*>(tab + (size_t)r.row[j] * 2);
          v[i][j][0] = q.x;
          v[i][j][FW > 1 ? 1 : 0] = q.y;
        } else if (FW == 4) {
          const uint4 q = *reinterpret_cast<const uint4*>(tab + (size_t)r.row[j] * 4);
          v[i][j][0] = q.x;
          v[i][j][FW > 1 ? 1 : 0] = q.y;
          v[i][j][FW > 2 ? 2 : 0] = q.z;
          v[i][j][FW > 3 ? 3 : 0] = q.w;
        } else {
#pragma unroll
          for (int f = 0; f < FW; ++f) v[i][j][f] = tab[(size_t)r.row[j] * FW + f];
        }
      }
      weights_d3(fr, w[i]);
    }
#pragma unroll
    for (int i = 0; i < PPT; ++i)
#pragma unroll
      for (int f = 0; f < FW; ++f) {
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          a0 = a0 + w[i][j] * TT::to_f32((uint16_t)(v[i][j][f] & 0xffffu));
          a1 = a1 + w[i][j] * TT::to_f32((uint16_t)(v[i][j][f] >> 16));
        }
        stage[(l * FW + f) * LD + t + TILE_THREADS * i] = TT::pack(a0, a1);
      }
  }
  __syncthreads();

  // Each point's L*FW*4 bytes leave as pieces of 16 bytes; consecutive lanes take
  // consecutive pieces, so a wave writes 1 KiB of contiguous output per instruction.
  const int pieces = (L * FW) >> 2;
  const int total = P * pieces;
  for (int c = t; c < total; c += TILE_THREADS) {
    const int p = c / pieces, q = c - p * pieces;
    const int64_t n = p0 + p;
    if (n < N) {
      uint4 val;
      val.x = stage[(4 * q + 0) * LD + p];
      val.y = stage[(4 * q + 1) * LD + p];
      val.z = stage[(4 * q + 2) * LD + p];
      val.w = stage[(4 * q + 3) * LD + p];
      *reinterpret_cast<uint4*>(out + n * out_stride + 8 * q) = val;
    }
  }
}

// Level sweep: the same work with (nearly) the whole grid resident at once.  A thread keeps the packed results of all
// its PPT points' levels in registers and stores finished 64-byte rows at the end; nothing is staged in LDS, so three
// or four workgroups fit a CU and a million points take little more than one round of workgroups.  Workgroups
// that start together and do the same work per level stay together: at any moment an XCD's L2 serves the gathers of
// a few level tables, not of all of them (a workgroup that runs ahead fetches cold lines and falls back, one
// that lags finds them warm and catches up).  With workgroups that start at different times, as in the staged
// kernel's several rounds, every level's table competes for L2 at once.  (Perfect lock-step is not the aim: one
// workgroup per CU, all in the same phase of the same level, lets the memory pipeline drain at every level.)
template <typename TT, int PPT, int D, bool LDS0 = false>
__global__ __launch_bounds__(TILE_THREADS) void hash_fwd_sweep_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                                 const uint32_t* table, uint16_t* out, int64_t out_stride,
                                                                 int64_t N, DevGeom g, const int64_t* primes, float scale) {
  constexpr int P = TILE_THREADS * PPT;
  constexpr int LMAX = 16;
  const int t = threadIdx.x;
  const int64_t p0 = (int64_t)blockIdx.x * P;
  const int L = g.levels;
  float x[PPT][3];
#pragma unroll
  for (int i = 0; i < PPT; ++i) {
    int64_t n = p0 + t + TILE_THREADS * i;
    if (n >= N) n = N - 1;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      float v = load_as_f32(coords, n * csn + d * csd, cdt);
      x[i][d] = scale != 1.0f ? v / scale : v;
    }
  }
  // LDS0: the rows of level 0 (dense, a few thousand) are copied to LDS once per workgroup and gathered from there
  extern __shared__ uint32_t level0_rows[];
  if constexpr (LDS0) {
    const uint32_t* src = table + g.row_offset[0];
    for (uint32_t i = t; i < g.rows[0]; i += TILE_THREADS) level0_rows[i] = src[i];
    __syncthreads();
  }
  constexpr int CN = 1 << D;  // corners of a cell
  const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], D > 2 ? (uint32_t)primes[D > 2 ? 2 : 0] : 0u};
  uint32_t enc[PPT][LMAX];
#pragma unroll
  for (int l = 0; l < LMAX; ++l) {
    if (l < L) {
      const uint32_t res = (uint32_t)g.res[l];
      const float fres = (float)g.res[l];
      const bool hashed = l >= g.first_hash;
      const uint32_t mask = g.rows[l] - 1;
      const uint32_t* tab = table + g.row_offset[l];
#pragma unroll
      for (int i0 = 0; i0 < PPT; i0 += 2) {
        uint32_t v[2][8];
        float w[2][8];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          uint32_t c[3];
          float fr[3];
#pragma unroll
          for (int d = 0; d < D; ++d) {
            const float pos = x[i0 + i][d] * fres;
            const float fl = floorf(pos);
            c[d] = cell_index(fl, fres);
            fr[d] = pos - fl;
          }
          const Corner8 r = D == 3 ? rows_d3(c, hashed, res, mask, pi) : rows_d2(c, hashed, res, mask, pi);
#pragma unroll
          for (int j = 0; j < CN; ++j) v[i][j] = (LDS0 && l == 0) ? level0_rows[r.row[j]] : tab[r.row[j]];
          if (D == 3) weights_d3(fr, w[i]);
          else weights_d2(fr, w[i]);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
          for (int j = 0; j < CN; ++j) {
            a0 = a0 + w[i][j] * TT::to_f32((uint16_t)(v[i][j] & 0xffffu));
            a1 = a1 + w[i][j] * TT::to_f32((uint16_t)(v[i][j] >> 16));
          }
          enc[i0 + i][l] = TT::pack(a0, a1);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < PPT; ++i) enc[i][l] = 0u;
    }
  }
#pragma unroll
  for (int i = 0; i < PPT; ++i) {
    const int64_t n = p0 + t + TILE_THREADS * i;
    if (n >= N) continue;
    uint4* dst = reinterpret_cast<uint4*>(out + n * out_stride);
#pragma unroll
    for (int q = 0; q < LMAX / 4; ++q)
      if (4 * q < L) dst[q] = make_uint4(enc[i][4 * q], enc[i][4 * q + 1], enc[i][4 * q + 2], enc[i][4 * q + 3]);
  }
}

// The level sweep for float32 tables (a row is one 8-byte pair, an output row 32 floats): same walk, same operation
// order as the per-(point, level) kernel, the results of a thread's PPT points held as float pairs.
template <int PPT>
__global__ __launch_bounds__(TILE_THREADS) void hash_fwd_sweep32_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                                   const float2* table, float* out, int64_t out_stride,
                                                                   int64_t N, DevGeom g, const int64_t* primes, float scale) {
  constexpr int P = TILE_THREADS * PPT;
  constexpr int LMAX = 16;
  const int t = threadIdx.x;
  const int64_t p0 = (int64_t)blockIdx.x * P;
  const int L = g.levels;
  float x[PPT][3];
#pragma unroll
  for (int i = 0; i < PPT; ++i) {
    int64_t n = p0 + t + TILE_THREADS * i;
    if (n >= N) n = N - 1;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
      float v = load_as_f32(coords, n * csn + d * csd, cdt);
      x[i][d] = scale != 1.0f ? v / scale : v;
    }
  }
  const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], (uint32_t)primes[2]};
  float2 enc[PPT][LMAX];
#pragma unroll
  for (int l = 0; l < LMAX; ++l) {
    if (l < L) {
      const uint32_t res = (uint32_t)g.res[l];
      const float fres = (float)g.res[l];
      const bool hashed = l >= g.first_hash;
      const uint32_t mask = g.rows[l] - 1;
      const float2* tab = table + g.row_offset[l];
      float2 v[PPT][8];
      float w[PPT][8];
#pragma unroll
      for (int i = 0; i < PPT; ++i) {
        uint32_t c[3];
        float fr[3];
#pragma unroll
        for (int d = 0; d < 3; ++d) {
          const float pos = x[i][d] * fres;
          const float fl = floorf(pos);
          c[d] = cell_index(fl, fres);
          fr[d] = pos - fl;
        }
        const Corner8 r = rows_d3(c, hashed, res, mask, pi);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = tab[r.row[j]];
        weights_d3(fr, w[i]);
      }
#pragma unroll
      for (int i = 0; i < PPT; ++i) {
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          a0 = a0 + w[i][j] * v[i][j].x;
          a1 = a1 + w[i][j] * v[i][j].y;
        }
        enc[i][l] = make_float2(a0, a1);
      }
    } else {
#pragma unroll
      for (int i = 0; i < PPT; ++i) enc[i][l] = make_float2(0.0f, 0.0f);
    }
  }
#pragma unroll
  for (int i = 0; i < PPT; ++i) {
    const int64_t n = p0 + t + TILE_THREADS * i;
    if (n >= N) continue;
    float4* dst = reinterpret_cast<float4*>(out + n * out_stride);
#pragma unroll
    for (int q = 0; q < LMAX / 2; ++q)
      if (2 * q < L) dst[q] = make_float4(enc[i][2 * q].x, enc[i][2 * q].y, enc[i][2 * q + 1].x, enc[i][2 * q + 1].y);
  }
}

template <typename GT, int PPT>
__global__ __launch_bounds__(TILE_THREADS) void hash_bwd_tiled_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                                 const uint16_t* dout, int64_t dout_stride,
                                                                 float* dtable, int64_t N, DevGeom g,
                                                                 const int64_t* primes, float scale) {
  constexpr int P = TILE_THREADS * PPT;
  constexpr int LD = P + 2;
  extern __shared__ uint32_t stage[];
  const int t = threadIdx.x;
  const int64_t p0 = (int64_t)blockIdx.x * P;
  const int L = g.levels;

  const int pieces = L >> 2;
  const int total = P * pieces;
  for (int c = t; c < total; c += TILE_THREADS) {
    const int p = c / pieces, q = c - p * pieces;
    const int64_t n = p0 + p;
    uint4 val = make_uint4(0u, 0u, 0u, 0u);
    if (n < N) val = *reinterpret_cast<const uint4*>(dout + n * dout_stride + 8 * q);
    stage[(4 * q + 0) * LD + p] = val.x;
    stage[(4 * q + 1) * LD + p] = val.y;
    stage[(4 * q + 2) * LD + p] = val.z;
    stage[(4 * q + 3) * LD + p] = val.w;
  }

  float x[PPT][3];
  bool valid[PPT];
#pragma unroll
  for (int i = 0; i < PPT; ++i) {
    int64_t n = p0 + t + TILE_THREADS * i;
    valid[i] = n < N;
    if (n >= N) n = N - 1;
#pragma unroll
    for (int d = 0; d < 3; ++d) {
      float v = load_as_f32(coords, n * csn + d * csd, cdt);
      x[i][d] = scale != 1.0f ? v / scale : v;
    }
  }
  const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], (uint32_t)primes[2]};
  __syncthreads();

  for (int l = 0; l < L; ++l) {
    const uint32_t res = (uint32_t)g.res[l];
    const float fres = (float)g.res[l];
    const bool hashed = l >= g.first_hash;
    const uint32_t mask = g.rows[l] - 1;
    float* tab = dtable + g.row_offset[l] * 2;
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const uint32_t packed = stage[l * LD + t + TILE_THREADS * i];
      // a zero upstream gradient (both features) contributes nothing
      if (!valid[i] || (packed & 0x7fff7fffu) == 0u) continue;
      const float g0 = GT::to_f32((uint16_t)(packed & 0xffffu));
      const float g1 = GT::to_f32((uint16_t)(packed >> 16));
      uint32_t c[3];
      float fr[3];
#pragma unroll
      for (int d = 0; d < 3; ++d) {
        const float pos = x[i][d] * fres;
        const float fl = floorf(pos);
        c[d] = cell_index(fl, fres);
        fr[d] = pos - fl;
      }
      const Corner8 r = rows_d3(c, hashed, res, mask, pi);
      float w[8];
      weights_d3(fr, w);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float* dst = tab + 2 * (size_t)r.row[j];
        unsafeAtomicAdd(dst, w[j] * g0);
        unsafeAtomicAdd(dst + 1, w[j] * g1);
      }
    }
  }
}

// Small batches: one thread per (point, level), the levels of a point side by side in blockIdx.y.  A thread per point
// walks its levels one after the other, and a batch of a few thousand points is then a handful of workgroups that wait
// out sixteen rounds of memory latency (forward) or queue five hundred atomics per thread behind each other (backward)
// while most of the chip idles.  Same arithmetic, in the same order, as the kernels above.
template <typename TT, int D>
__global__ __launch_bounds__(TILE_THREADS) void hash_fwd_level_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                                 const uint32_t* table, uint16_t* out, int64_t out_stride,
                                                                 int64_t N, DevGeom g, const int64_t* primes, float scale) {
  const int l = blockIdx.y;
  const int64_t n = (int64_t)blockIdx.x * TILE_THREADS + threadIdx.x;
  if (n >= N) return;
  constexpr int CN = 1 << D;
  const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], D > 2 ? (uint32_t)primes[D > 2 ? 2 : 0] : 0u};
  const uint32_t res = (uint32_t)g.res[l];
  const float fres = (float)g.res[l];
  const uint32_t* tab = table + g.row_offset[l];
  uint32_t c[3];
  float fr[3];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    float v = load_as_f32(coords, n * csn + d * csd, cdt);
    v = scale != 1.0f ? v / scale : v;
    const float pos = v * fres;
    const float fl = floorf(pos);
    c[d] = cell_index(fl, fres);
    fr[d] = pos - fl;
  }
  const Corner8 r = D == 3 ? rows_d3(c, l >= g.first_hash, res, g.rows[l] - 1, pi) : rows_d2(c, l >= g.first_hash, res, g.rows[l] - 1, pi);
  uint32_t v[CN];
#pragma unroll
  for (int j = 0; j < CN; ++j) v[j] = tab[r.row[j]];
  float w[8];
  if (D == 3) weights_d3(fr, w);
  else weights_d2(fr, w);
  float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
  for (int j = 0; j < CN; ++j) {
    a0 = a0 + w[j] * TT::to_f32((uint16_t)(v[j] & 0xffffu));
    a1 = a1 + w[j] * TT::to_f32((uint16_t)(v[j] >> 16));
  }
  *reinterpret_cast<uint32_t*>(out + n * out_stride + 2 * l) = TT::pack(a0, a1);
}

template <typename GT, int D>
__global__ __launch_bounds__(TILE_THREADS) void hash_bwd_level_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                                 const uint16_t* dout, int64_t dout_stride, float* dtable,
                                                                 int64_t N, DevGeom g, const int64_t* primes, float scale) {
  const int l = blockIdx.y;
  const int64_t n = (int64_t)blockIdx.x * TILE_THREADS + threadIdx.x;
  if (n >= N) return;
  const uint32_t packed = *reinterpret_cast<const uint32_t*>(dout + n * dout_stride + 2 * l);
  // a zero upstream gradient (both features) contributes nothing
  if ((packed & 0x7fff7fffu) == 0u) return;
  constexpr int CN = 1 << D;
  const float g0 = GT::to_f32((uint16_t)(packed & 0xffffu));
  const float g1 = GT::to_f32((uint16_t)(packed >> 16));
  const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], D > 2 ? (uint32_t)primes[D > 2 ? 2 : 0] : 0u};
  const uint32_t res = (uint32_t)g.res[l];
  const float fres = (float)g.res[l];
  float* tab = dtable + g.row_offset[l] * 2;
  uint32_t c[3];
  float fr[3];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    float v = load_as_f32(coords, n * csn + d * csd, cdt);
    v = scale != 1.0f ? v / scale : v;
    const float pos = v * fres;
    const float fl = floorf(pos);
    c[d] = cell_index(fl, fres);
    fr[d] = pos - fl;
  }
  const Corner8 r = D == 3 ? rows_d3(c, l >= g.first_hash, res, g.rows[l] - 1, pi) : rows_d2(c, l >= g.first_hash, res, g.rows[l] - 1, pi);
  float w[8];
  if (D == 3) weights_d3(fr, w);
  else weights_d2(fr, w);
#pragma unroll
  for (int j = 0; j < CN; ++j) {
    float* dst = tab + 2 * (size_t)r.row[j];
    unsafeAtomicAdd(dst, w[j] * g0);
    unsafeAtomicAdd(dst + 1, w[j] * g1);
  }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
// below this many points the scattered-atomic kernels are faster than planning + scanning
constexpr int64_t SCAN_MIN_POINTS = 32768;
constexpr int64_t BIN_MIN_POINTS = 8192;  // below: the sort's fixed cost (about 100 us) exceeds the scattered atomics' 13 ns per point
constexpr int SWEEP_PPT = 4;
constexpr int64_t SWEEP_MIN_POINTS = (int64_t)256 * TILE_THREADS * SWEEP_PPT;
// the forward per (point, level) serves batches up to this where the staged kernel is the alternative (three
// dimensions: 45 against 53 us at 2^16 points, 75 against 52 us at 2^17); in two dimensions up to the sweep's minimum
constexpr int64_t LEVEL_MAX_POINTS = 65536;

static bool tiled_ok(const nf_hash_geom* g, int table_dt, const void* rows_ptr, int64_t row_stride, int feat = 2, int dims = 3) {
  if (g->dims != dims || g->feat != feat || table_dt == NF_F32) return false;
  if ((g->levels * (feat / 2)) % 4 != 0 || g->levels > 16) return false;
  for (int l = g->first_hash_level; l < g->levels; ++l) {
    if (l < 0) return false;
    const int64_t r = g->rows[l];
    if ((r & (r - 1)) != 0) return false;
  }
  if (((uintptr_t)rows_ptr & 15u) != 0 || (row_stride * 2) % 16 != 0) return false;
  return true;
}

// the per-(point, level) kernels for small batches: rows of one 16-bit pair, two or three dimensions, hashed levels of
// a power of two of rows, pairs that can be read and written as one 32-bit word
static bool level_ok(const nf_hash_geom* g, int table_dt, const void* rows_ptr, int64_t row_stride) {
  if ((g->dims != 2 && g->dims != 3) || g->feat != 2 || table_dt == NF_F32) return false;
  for (int l = g->first_hash_level; l < g->levels; ++l) {
    if (l < 0) return false;
    const int64_t r = g->rows[l];
    if ((r & (r - 1)) != 0) return false;
  }
  return ((uintptr_t)rows_ptr & 3u) == 0 && row_stride % 2 == 0;
}

static bool sweep32_ok(const nf_hash_geom* g, const void* table, const void* rows_ptr, int64_t row_stride) {
  if (g->dims != 3 || g->feat != 2 || g->levels % 2 != 0 || g->levels > 16) return false;
  for (int l = g->first_hash_level; l < g->levels; ++l) {
    if (l < 0) return false;
    const int64_t r = g->rows[l];
    if ((r & (r - 1)) != 0) return false;
  }
  return ((uintptr_t)table & 7u) == 0 && ((uintptr_t)rows_ptr & 15u) == 0 && row_stride % 4 == 0;
}

template <int D, typename TT>
static void launch_fwd_generic(const void* coords, int cdt, int64_t csn, int64_t csd, const void* table, void* out,
                               int64_t out_stride, int64_t N, const DevGeom& g, const int64_t* primes, float scale, bool vec,
                               hipStream_t s) {
  typedef typename TT::storage S;
  dim3 grid((unsigned)((N + 255) / 256), (unsigned)g.levels);
  // the widest piece of 16, 8 or 4 bytes that divides a row and keeps every row of the table and of the output aligned
  int v = 1;
  if (vec && D <= 4)
    for (int bytes = 16; bytes > (int)sizeof(S); bytes >>= 1) {
      const int c = bytes / (int)sizeof(S);
      if (g.feat % c == 0 && out_stride % c == 0 && (uintptr_t)table % bytes == 0 && (uintptr_t)out % bytes == 0) {
        v = c;
        break;
      }
    }
  const void* kern = (const void*)hash_fwd_generic_k<D, TT, 1>;
  if constexpr (D <= 4) {
    if (v == 2) kern = (const void*)hash_fwd_generic_k<D, TT, 2>;
    if (v == 4) kern = (const void*)hash_fwd_generic_k<D, TT, 4>;
    if constexpr (sizeof(S) == 2)
      if (v == 8) kern = (const void*)hash_fwd_generic_k<D, TT, 8>;
  }
  const S* tab = (const S*)table;
  S* o = (S*)out;
  DevGeom gg = g;
  void* args[] = {&coords, &cdt, &csn, &csd, &tab, &o, &out_stride, &N, &gg, &primes, &scale};
  (void)hipLaunchKernel(kern, grid, dim3(256), args, 0, s);  // the caller reads the launch status
}

template <int D>
static int dispatch_fwd_generic(int table_dt, const void* coords, int cdt, int64_t csn, int64_t csd, const void* table,
                                void* out, int64_t out_stride, int64_t N, const DevGeom& g, const int64_t* primes,
                                float scale, bool vec, hipStream_t s) {
  switch (table_dt) {
    case NF_F32: launch_fwd_generic<D, F32>(coords, cdt, csn, csd, table, out, out_stride, N, g, primes, scale, vec, s); break;
    case NF_F16: launch_fwd_generic<D, F16>(coords, cdt, csn, csd, table, out, out_stride, N, g, primes, scale, vec, s); break;
    default: launch_fwd_generic<D, BF16>(coords, cdt, csn, csd, table, out, out_stride, N, g, primes, scale, vec, s); break;
  }
  return check_launch("hash_fwd_generic");
}

template <int FW>
static int launch_fwd_tiled_wide(int table_dtype, const void* coords, int coords_dtype, int64_t csn, int64_t csd, const void* table,
                                 void* out, int64_t out_stride_n, int64_t n_points, const DevGeom& g, const int64_t* primes,
                                 float scale, hipStream_t s) {
  constexpr int PPT = FW <= 2 ? 2 : 1;
  constexpr int P = TILE_THREADS * PPT;
  const size_t lds = (size_t)g.levels * FW * (P + 2) * sizeof(uint32_t);
  dim3 grid((unsigned)((n_points + P - 1) / P));
  const void* kern = table_dtype == NF_F16 ? (const void*)hash_fwd_tiled_k<F16, PPT, FW> : (const void*)hash_fwd_tiled_k<BF16, PPT, FW>;
  if (lds > 64 * 1024) {
    const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  const uint32_t* tab = (const uint32_t*)table;
  uint16_t* o = (uint16_t*)out;
  void* args[] = {(void*)&coords, (void*)&coords_dtype, (void*)&csn, (void*)&csd, (void*)&tab, (void*)&o,
                  (void*)&out_stride_n, (void*)&n_points, (void*)&g, (void*)&primes, (void*)&scale};
  const hipError_t e = hipLaunchKernel(kern, grid, dim3(TILE_THREADS), args, lds, s);
  if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(hash_fwd_tiled): %s", hipGetErrorString(e));
  return check_launch("hash_fwd_tiled");
}

}  // namespace nf

using namespace nf;

extern "C" int nf_hash_encode_fwd(const void* coords, int coords_dtype, int64_t csn, int64_t csd, const void* table,
                                  int table_dtype, void* out, int64_t out_stride_n, int64_t n_points,
                                  const nf_hash_geom* geom, const int64_t* primes, float scale, int flags,
                                  void* stream) {
  DevGeom g;
  if (int rc = make_dev_geom(geom, &g)) return rc;
  NF_REQUIRE(dtype_ok(coords_dtype) && dtype_ok(table_dtype), NF_EINVAL, "unknown dtype code");
  NF_REQUIRE(n_points >= 0, NF_EINVAL, "n_points negative");
  NF_REQUIRE(out_stride_n >= (int64_t)g.levels * g.feat, NF_EINVAL, "out_stride_n=%lld < levels*feat",
             (long long)out_stride_n);
  NF_REQUIRE(scale > 0.0f, NF_EINVAL, "scale must be positive");
  if (n_points == 0) return 0;
  NF_REQUIRE(coords && table && out && primes, NF_EINVAL, "NULL pointer argument");
  NF_REQUIRE(n_points <= ((int64_t)1 << 31) * 256 - 1, NF_EINVAL, "n_points too large");
  hipStream_t s = (hipStream_t)stream;

  // More than sixteen levels: the fast kernels keep a point's results of up to sixteen levels in registers, and the
  // levels are independent, so the call runs as one call per sixteen levels on its own columns of the output
  // (2^20 points, 32 levels: 1.03 -> 0.73 ms).
  if (g.levels > 16 && !(flags & NF_HASH_FORCE_GENERIC)) {
    for (int l0 = 0; l0 < g.levels; l0 += 16) {
      nf_hash_geom part = *geom;
      part.levels = g.levels - l0 < 16 ? g.levels - l0 : 16;
      const int fh = geom->first_hash_level - l0;
      part.first_hash_level = fh < 0 ? 0 : (fh > part.levels ? part.levels : fh);
      for (int l = 0; l < part.levels; ++l) {
        part.res[l] = geom->res[l0 + l];
        part.rows[l] = geom->rows[l0 + l];
        part.row_offset[l] = geom->row_offset[l0 + l];
      }
      void* cols = (char*)out + (size_t)l0 * g.feat * dtype_size(table_dtype);
      if (int rc = nf_hash_encode_fwd(coords, coords_dtype, csn, csd, table, table_dtype, cols, out_stride_n, n_points, &part, primes, scale,
                                      flags, stream))
        return rc;
    }
    return 0;
  }

  // float32 tables: the same sweep on 8-byte rows
  if (!(flags & (NF_HASH_FORCE_GENERIC | NF_HASH_FWD_STAGED)) && n_points >= SWEEP_MIN_POINTS && table_dtype == NF_F32 &&
      sweep32_ok(geom, table, out, out_stride_n)) {
    constexpr int PPT = 2;
    constexpr int P = TILE_THREADS * PPT;
    // launches of 1024 workgroups (2^19 points), for the reason given at the 16-bit sweep below
    // (2^20 points: 663 -> 613 us, 2^22 points: 3514 -> 2687 us)
    constexpr int64_t CHUNK = (int64_t)1024 * P;
    for (int64_t n0 = 0; n0 < n_points; n0 += CHUNK) {
      const int64_t n = n_points - n0 < CHUNK ? n_points - n0 : CHUNK;
      const void* c = (const char*)coords + n0 * csn * dtype_size(coords_dtype);
      hipLaunchKernelGGL((hash_fwd_sweep32_k<PPT>), dim3((unsigned)((n + P - 1) / P)), dim3(TILE_THREADS), 0, s, c, coords_dtype, csn,
                         csd, (const float2*)table, (float*)out + n0 * out_stride_n, out_stride_n, n, g, primes, scale);
    }
    return check_launch("hash_fwd_sweep32");
  }
  // The level sweep wants at least one workgroup per compute unit; below that the staged kernel's smaller tiles
  // spread the points over more of the chip.
  if (!(flags & (NF_HASH_FORCE_GENERIC | NF_HASH_FWD_STAGED)) && n_points >= SWEEP_MIN_POINTS &&
      tiled_ok(geom, table_dtype, out, out_stride_n)) {
    constexpr int PPT = SWEEP_PPT;
    constexpr int P = TILE_THREADS * PPT;
    // level 0 in LDS where it is dense and small (19.6 KB at resolution 16): worth about 1 % (its rows mostly hit L1 anyway)
    const bool lds0 = geom->first_hash_level > 0 && geom->rows[0] * 4 <= 32 * 1024;
    const size_t lds = lds0 ? (size_t)geom->rows[0] * 4 : 0;
    const void* kern = table_dtype == NF_F16 ? (lds0 ? (const void*)hash_fwd_sweep_k<F16, PPT, 3, true> : (const void*)hash_fwd_sweep_k<F16, PPT, 3>)
                                             : (lds0 ? (const void*)hash_fwd_sweep_k<BF16, PPT, 3, true> : (const void*)hash_fwd_sweep_k<BF16, PPT, 3>);
    const uint32_t* tab = (const uint32_t*)table;
    // Launches of at most 2^20 points: the workgroups of one launch are (nearly) all resident and walk the levels
    // together; in one launch of 2^22 points later rounds of workgroups meet earlier ones at other levels and the
    // tables compete for L2 (1545 us against 1324 us in four launches; 677 against 661 us at 2^21).
    constexpr int64_t CHUNK = (int64_t)1 << 20;
    for (int64_t n0 = 0; n0 < n_points; n0 += CHUNK) {
      const int64_t n = n_points - n0 < CHUNK ? n_points - n0 : CHUNK;
      const void* c = (const char*)coords + n0 * csn * dtype_size(coords_dtype);
      uint16_t* o = (uint16_t*)out + n0 * out_stride_n;
      void* args[] = {(void*)&c, (void*)&coords_dtype, (void*)&csn, (void*)&csd, (void*)&tab, (void*)&o, (void*)&out_stride_n,
                      (void*)&n, (void*)&g, (void*)&primes, (void*)&scale};
      const hipError_t e = hipLaunchKernel(kern, dim3((unsigned)((n + P - 1) / P)), dim3(TILE_THREADS), args, lds, s);
      if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(hash_fwd_sweep): %s", hipGetErrorString(e));
    }
    return check_launch("hash_fwd_sweep");
  }
  // two dimensions: the same sweep over four corners
  if (!(flags & (NF_HASH_FORCE_GENERIC | NF_HASH_FWD_STAGED)) && n_points >= SWEEP_MIN_POINTS &&
      tiled_ok(geom, table_dtype, out, out_stride_n, 2, 2)) {
    constexpr int PPT = SWEEP_PPT;
    constexpr int P = TILE_THREADS * PPT;
    dim3 grid((unsigned)((n_points + P - 1) / P));
    if (table_dtype == NF_F16)
      hipLaunchKernelGGL((hash_fwd_sweep_k<F16, PPT, 2>), grid, dim3(TILE_THREADS), 0, s, coords, coords_dtype, csn, csd,
                         (const uint32_t*)table, (uint16_t*)out, out_stride_n, n_points, g, primes, scale);
    else
      hipLaunchKernelGGL((hash_fwd_sweep_k<BF16, PPT, 2>), grid, dim3(TILE_THREADS), 0, s, coords, coords_dtype, csn, csd,
                         (const uint32_t*)table, (uint16_t*)out, out_stride_n, n_points, g, primes, scale);
    return check_launch("hash_fwd_sweep");
  }
  // batches below the sweep's minimum: a thread per (point, level)
  if (!(flags & (NF_HASH_FORCE_GENERIC | NF_HASH_FWD_STAGED)) && level_ok(geom, table_dtype, out, out_stride_n) &&
      (n_points <= LEVEL_MAX_POINTS || !tiled_ok(geom, table_dtype, out, out_stride_n))) {
    dim3 grid((unsigned)((n_points + TILE_THREADS - 1) / TILE_THREADS), (unsigned)g.levels);
    const void* kern = table_dtype == NF_F16 ? (g.dims == 3 ? (const void*)hash_fwd_level_k<F16, 3> : (const void*)hash_fwd_level_k<F16, 2>)
                                             : (g.dims == 3 ? (const void*)hash_fwd_level_k<BF16, 3> : (const void*)hash_fwd_level_k<BF16, 2>);
    const uint32_t* tab = (const uint32_t*)table;
    uint16_t* o = (uint16_t*)out;
    void* args[] = {&coords, &coords_dtype, &csn, &csd, &tab, &o, &out_stride_n, &n_points, &g, &primes, &scale};
    const hipError_t e = hipLaunchKernel(kern, grid, dim3(TILE_THREADS), args, 0, s);
    if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(hash_fwd_level): %s", hipGetErrorString(e));
    return check_launch("hash_fwd_level");
  }
  if (!(flags & NF_HASH_FORCE_GENERIC) && tiled_ok(geom, table_dtype, out, out_stride_n)) {
    constexpr int PPT = 2;
    constexpr int P = TILE_THREADS * PPT;
    const size_t lds = (size_t)g.levels * (P + 2) * sizeof(uint32_t);
    dim3 grid((unsigned)((n_points + P - 1) / P));
    if (table_dtype == NF_F16)
      hipLaunchKernelGGL((hash_fwd_tiled_k<F16, PPT, 1>), grid, dim3(TILE_THREADS), lds, s, coords, coords_dtype, csn,
                         csd, (const uint32_t*)table, (uint16_t*)out, out_stride_n, n_points, g, primes, scale);
    else
      hipLaunchKernelGGL((hash_fwd_tiled_k<BF16, PPT, 1>), grid, dim3(TILE_THREADS), lds, s, coords, coords_dtype, csn,
                         csd, (const uint32_t*)table, (uint16_t*)out, out_stride_n, n_points, g, primes, scale);
    return check_launch("hash_fwd_tiled");
  }
  // 16-bit rows of 4 or 8 features: the staged kernel with 8- or 16-byte gathers
  if (!(flags & NF_HASH_FORCE_GENERIC) && (geom->feat == 4 || geom->feat == 8) && tiled_ok(geom, table_dtype, out, out_stride_n, geom->feat) &&
      ((uintptr_t)table % (2 * geom->feat) == 0)) {
    return geom->feat == 4 ? launch_fwd_tiled_wide<2>(table_dtype, coords, coords_dtype, csn, csd, table, out, out_stride_n, n_points, g, primes, scale, s)
                           : launch_fwd_tiled_wide<4>(table_dtype, coords, coords_dtype, csn, csd, table, out, out_stride_n, n_points, g, primes, scale, s);
  }
  const bool vec = !(flags & NF_HASH_FORCE_GENERIC);  // the flag keeps the scalar form as the other kernels' bit-exact check
  switch (g.dims) {
    case 1: return dispatch_fwd_generic<1>(table_dtype, coords, coords_dtype, csn, csd, table, out, out_stride_n, n_points, g, primes, scale, vec, s);
    case 2: return dispatch_fwd_generic<2>(table_dtype, coords, coords_dtype, csn, csd, table, out, out_stride_n, n_points, g, primes, scale, vec, s);
    case 3: return dispatch_fwd_generic<3>(table_dtype, coords, coords_dtype, csn, csd, table, out, out_stride_n, n_points, g, primes, scale, vec, s);
    case 4: return dispatch_fwd_generic<4>(table_dtype, coords, coords_dtype, csn, csd, table, out, out_stride_n, n_points, g, primes, scale, vec, s);
    case 5: return dispatch_fwd_generic<5>(table_dtype, coords, coords_dtype, csn, csd, table, out, out_stride_n, n_points, g, primes, scale, vec, s);
    default: return dispatch_fwd_generic<6>(table_dtype, coords, coords_dtype, csn, csd, table, out, out_stride_n, n_points, g, primes, scale, vec, s);
  }
}

// whether a batch is large enough for one of the backward's LDS-tile variants
static bool bwd_tiles_apply(int64_t n_points, const nf_hash_geom* geom, int flags) {
  if (flags & NF_HASH_FORCE_PLANES) return n_points >= SCAN_MIN_POINTS;
  return n_points >= BIN_MIN_POINTS || bwd_direct_applies(n_points, geom, flags);
}

extern "C" int64_t nf_hash_encode_bwd_workspace_bytes(int64_t n_points, const nf_hash_geom* geom, int dout_dtype, int flags) {
  if (geom == nullptr || (flags & (NF_HASH_FORCE_GENERIC | NF_HASH_FORCE_ATOMIC))) return 0;
  if (!bwd_tiles_apply(n_points, geom, flags)) return 0;
  const int64_t scan = n_points >= SCAN_MIN_POINTS ? bwd_scan_workspace_bytes(n_points, geom, dout_dtype) : 0;
  if (flags & NF_HASH_FORCE_PLANES) return scan;
  const int64_t bin = bwd_bin_workspace_bytes(n_points, geom, dout_dtype, flags);
  return bin > 0 ? bin : scan;  // the bit-planes are what runs where the other kernels do not cover the geometry
}

extern "C" int nf_hash_encode_bwd(const void* coords, int coords_dtype, int64_t csn, int64_t csd, const void* dout,
                                  int dout_dtype, int64_t dout_stride_n, float* dtable, int64_t n_points,
                                  const nf_hash_geom* geom, const int64_t* primes, float scale, void* workspace,
                                  int64_t workspace_bytes, int flags, void* stream) {
  DevGeom g;
  if (int rc = make_dev_geom(geom, &g)) return rc;
  NF_REQUIRE(dtype_ok(coords_dtype) && dtype_ok(dout_dtype), NF_EINVAL, "unknown dtype code");
  NF_REQUIRE(n_points >= 0, NF_EINVAL, "n_points negative");
  NF_REQUIRE(dout_stride_n >= (int64_t)g.levels * g.feat, NF_EINVAL, "dout_stride_n=%lld < levels*feat",
             (long long)dout_stride_n);
  NF_REQUIRE(scale > 0.0f, NF_EINVAL, "scale must be positive");
  if (n_points == 0) return 0;
  NF_REQUIRE(coords && dout && dtable && primes, NF_EINVAL, "NULL pointer argument");
  NF_REQUIRE(n_points <= ((int64_t)1 << 31) * 256 - 1, NF_EINVAL, "n_points too large");
  hipStream_t s = (hipStream_t)stream;

  // large batches: accumulate in LDS tiles (needs the caller's workspace for the sorted records or the bit-planes)
  if (!(flags & (NF_HASH_FORCE_GENERIC | NF_HASH_FORCE_ATOMIC)) && workspace != nullptr &&
      bwd_tiles_apply(n_points, geom, flags) &&
      ((uintptr_t)dout % (dout_dtype == NF_F32 ? 8 : 4) == 0) && (dout_stride_n % 2 == 0) && ((uintptr_t)workspace % 4 == 0)) {
    const int64_t need_bin = bwd_bin_workspace_bytes(n_points, geom, dout_dtype, flags);
    if (!(flags & NF_HASH_FORCE_PLANES) && need_bin > 0 && workspace_bytes >= need_bin && ((uintptr_t)workspace % 16 == 0))
      return launch_bwd_bin(coords, coords_dtype, csn, csd, dout, dout_dtype, dout_stride_n, dtable, n_points, geom, g, primes,
                            scale, workspace, flags, s);
    const int64_t need = n_points >= SCAN_MIN_POINTS ? bwd_scan_workspace_bytes(n_points, geom, dout_dtype) : 0;
    if (need > 0 && workspace_bytes >= need)
      return launch_bwd_scan(coords, coords_dtype, csn, csd, dout, dout_dtype, dout_stride_n, dtable, n_points, geom, g,
                             primes, scale, workspace, s);
  }
  // small batches: a thread per (point, level)
  if (!(flags & NF_HASH_FORCE_GENERIC) && level_ok(geom, dout_dtype, dout, dout_stride_n) &&
      (n_points < BIN_MIN_POINTS || !tiled_ok(geom, dout_dtype, dout, dout_stride_n))) {
    dim3 grid((unsigned)((n_points + TILE_THREADS - 1) / TILE_THREADS), (unsigned)g.levels);
    const void* kern = dout_dtype == NF_F16 ? (g.dims == 3 ? (const void*)hash_bwd_level_k<F16, 3> : (const void*)hash_bwd_level_k<F16, 2>)
                                            : (g.dims == 3 ? (const void*)hash_bwd_level_k<BF16, 3> : (const void*)hash_bwd_level_k<BF16, 2>);
    const uint16_t* d = (const uint16_t*)dout;
    void* args[] = {&coords, &coords_dtype, &csn, &csd, &d, &dout_stride_n, &dtable, &n_points, &g, &primes, &scale};
    const hipError_t e = hipLaunchKernel(kern, grid, dim3(TILE_THREADS), args, 0, s);
    if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(hash_bwd_level): %s", hipGetErrorString(e));
    return check_launch("hash_bwd_level");
  }
  if (!(flags & NF_HASH_FORCE_GENERIC) && tiled_ok(geom, dout_dtype, dout, dout_stride_n)) {
    constexpr int PPT = 2;
    constexpr int P = TILE_THREADS * PPT;
    const size_t lds = (size_t)g.levels * (P + 2) * sizeof(uint32_t);
    dim3 grid((unsigned)((n_points + P - 1) / P));
    if (dout_dtype == NF_F16)
      hipLaunchKernelGGL((hash_bwd_tiled_k<F16, PPT>), grid, dim3(TILE_THREADS), lds, s, coords, coords_dtype, csn,
                         csd, (const uint16_t*)dout, dout_stride_n, dtable, n_points, g, primes, scale);
    else
      hipLaunchKernelGGL((hash_bwd_tiled_k<BF16, PPT>), grid, dim3(TILE_THREADS), lds, s, coords, coords_dtype, csn,
                         csd, (const uint16_t*)dout, dout_stride_n, dtable, n_points, g, primes, scale);
    return check_launch("hash_bwd_tiled");
  }
  dim3 grid((unsigned)((n_points + 255) / 256), (unsigned)g.levels);
  switch (g.dims) {
    case 1: hipLaunchKernelGGL((hash_bwd_generic_k<1>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, dout, dout_dtype, dout_stride_n, dtable, n_points, g, primes, scale); break;
    case 2: hipLaunchKernelGGL((hash_bwd_generic_k<2>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, dout, dout_dtype, dout_stride_n, dtable, n_points, g, primes, scale); break;
    case 3: hipLaunchKernelGGL((hash_bwd_generic_k<3>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, dout, dout_dtype, dout_stride_n, dtable, n_points, g, primes, scale); break;
    case 4: hipLaunchKernelGGL((hash_bwd_generic_k<4>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, dout, dout_dtype, dout_stride_n, dtable, n_points, g, primes, scale); break;
    case 5: hipLaunchKernelGGL((hash_bwd_generic_k<5>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, dout, dout_dtype, dout_stride_n, dtable, n_points, g, primes, scale); break;
    default: hipLaunchKernelGGL((hash_bwd_generic_k<6>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, dout, dout_dtype, dout_stride_n, dtable, n_points, g, primes, scale); break;
  }
  return check_launch("hash_bwd_generic");
}

extern "C" int nf_hash_encode_indices_fast(const void* coords, int coords_dtype, int64_t csn, int64_t csd,
                                           int64_t* out_rows, float* out_w, int64_t n_points, const nf_hash_geom* geom,
                                           const int64_t* primes, float scale, void* stream) {
  DevGeom g;
  if (int rc = make_dev_geom(geom, &g)) return rc;
  NF_REQUIRE(dtype_ok(coords_dtype), NF_EINVAL, "unknown dtype code");
  NF_REQUIRE(n_points >= 0, NF_EINVAL, "n_points negative");
  NF_REQUIRE(scale > 0.0f, NF_EINVAL, "scale must be positive");
  NF_REQUIRE(g.dims == 2 || g.dims == 3, NF_EUNSUPPORTED, "the 32-bit index form covers 2 and 3 dimensions, got %d", g.dims);
  for (int l = g.first_hash < 0 ? 0 : g.first_hash; l < g.levels; ++l)
    NF_REQUIRE((g.rows[l] & (g.rows[l] - 1u)) == 0u, NF_EUNSUPPORTED,
               "the 32-bit index form needs power-of-two hashed levels (level %d has %u rows)", l, g.rows[l]);
  if (n_points == 0) return 0;
  NF_REQUIRE(coords && out_rows && primes, NF_EINVAL, "NULL pointer argument");
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)((n_points + 255) / 256), (unsigned)g.levels);
  if (g.dims == 3) hipLaunchKernelGGL((hash_indices_fast_k<3>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, out_rows, out_w, n_points, g, primes, scale);
  else hipLaunchKernelGGL((hash_indices_fast_k<2>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, out_rows, out_w, n_points, g, primes, scale);
  return check_launch("hash_indices_fast");
}

extern "C" int nf_hash_encode_indices(const void* coords, int coords_dtype, int64_t csn, int64_t csd,
                                      int64_t* out_rows, float* out_w, int64_t n_points, const nf_hash_geom* geom,
                                      const int64_t* primes, float scale, void* stream) {
  DevGeom g;
  if (int rc = make_dev_geom(geom, &g)) return rc;
  NF_REQUIRE(dtype_ok(coords_dtype), NF_EINVAL, "unknown dtype code");
  NF_REQUIRE(n_points >= 0, NF_EINVAL, "n_points negative");
  NF_REQUIRE(scale > 0.0f, NF_EINVAL, "scale must be positive");
  if (n_points == 0) return 0;
  NF_REQUIRE(coords && out_rows && primes, NF_EINVAL, "NULL pointer argument");
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)((n_points + 255) / 256), (unsigned)g.levels);
  switch (g.dims) {
    case 1: hipLaunchKernelGGL((hash_indices_k<1>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, out_rows, out_w, n_points, g, primes, scale); break;
    case 2: hipLaunchKernelGGL((hash_indices_k<2>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, out_rows, out_w, n_points, g, primes, scale); break;
    case 3: hipLaunchKernelGGL((hash_indices_k<3>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, out_rows, out_w, n_points, g, primes, scale); break;
    case 4: hipLaunchKernelGGL((hash_indices_k<4>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, out_rows, out_w, n_points, g, primes, scale); break;
    case 5: hipLaunchKernelGGL((hash_indices_k<5>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, out_rows, out_w, n_points, g, primes, scale); break;
    default: hipLaunchKernelGGL((hash_indices_k<6>), grid, dim3(256), 0, s, coords, coords_dtype, csn, csd, out_rows, out_w, n_points, g, primes, scale); break;
  }
  return check_launch("hash_indices");
}
