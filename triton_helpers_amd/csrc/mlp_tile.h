// Building blocks shared by the fused-MLP and reversible-MLP kernels (gfx950, wave64).
//
// All matmuls run on v_mfma_f32_16x16x32_{bf16,f16}.  Activations are kept
// "row-per-lane":   for a tile of 16 data rows, lane l = (n, g) with n = l % 16 the
// data row and g = l / 16 one of four lane groups.
//
//   * A layer computes  D^T = W * X^T :  A operand = weights (M = output feature),
//     B operand = activations (N = data row), so an accumulator tile `mt` leaves
//     lane (n, g) holding output features 16*mt + 4*g + r, r = 0..3, of row n.
//   * Packing those four values to 16 bit gives two dwords; the tiles 2*kc and
//     2*kc+1 together are exactly the B operand of K-chunk kc of the next layer,
//     provided the next layer's weights are laid out with the same K order
//     ("chain order", k_chain()).  No cross-lane traffic between layers.
//   * Operands that come straight from global memory use the natural K order
//     (k_nat()): lane (n, g) loads 8 consecutive features 32*kc + 8*g .. +7.
//
// Weights live in LDS as ready-made A fragments: fragment (mt, kc) is 64 lanes x
// 16 bytes, lane (m, g) holding W[16*mt + m][k(kc, g, 0..7)].
#pragma once

#include <type_traits>
#include "nf_common.h"

namespace nf {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

union Frag {
  uint4 u;
  uint32_t w[4];
  bf16x8_t b;
  f16x8_t h;
};

template <typename T>
__device__ __forceinline__ f32x4_t mfma16(const Frag& a, const Frag& b, f32x4_t c);
template <>
__device__ __forceinline__ f32x4_t mfma16<BF16>(const Frag& a, const Frag& b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4_t mfma16<F16>(const Frag& a, const Frag& b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, c, 0, 0, 0);
}

// K-slot -> feature maps (kc = 32-wide chunk, g = lane group, j = element 0..7)
__host__ __device__ __forceinline__ int k_nat(int kc, int g, int j) { return 32 * kc + 8 * g + j; }
__host__ __device__ __forceinline__ int k_chain(int kc, int g, int j) { return 32 * kc + 16 * (j >> 2) + 4 * g + (j & 3); }
// "Wide order" of the 16 outputs of accumulator tile mt: lane group g's four outputs of tiles 2p and 2p + 1 are the eight
// consecutive features 32p + 8g .. + 7 (one 16-byte access per lane and tile pair instead of two 8-byte ones); m = 4g + r.
__host__ __device__ __forceinline__ int wide_feature(int mt, int m) { return 32 * (mt >> 1) + 8 * (m >> 2) + 4 * (mt & 1) + (m & 3); }

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// Two floats -> one dword of 16-bit values, round-to-nearest-even, one v_cvt_pk_* instruction on gfx950.
template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <>
__device__ __forceinline__ uint32_t pack2<BF16>(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
template <>
__device__ __forceinline__ uint32_t pack2<F16>(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
}
template <typename T>
__device__ __forceinline__ float unpack_lo(uint32_t v);
template <typename T>
__device__ __forceinline__ float unpack_hi(uint32_t v);
template <>
__device__ __forceinline__ float unpack_lo<BF16>(uint32_t v) { return __uint_as_float(v << 16); }
template <>
__device__ __forceinline__ float unpack_hi<BF16>(uint32_t v) { return __uint_as_float(v & 0xffff0000u); }
template <>
__device__ __forceinline__ float unpack_lo<F16>(uint32_t v) { return (float)__builtin_bit_cast(f16x2_t, v)[0]; }
template <>
__device__ __forceinline__ float unpack_hi<F16>(uint32_t v) { return (float)__builtin_bit_cast(f16x2_t, v)[1]; }

// Normal CDF for GELU:  Phi(z) = 0.5 + z * Q(z^2), Q a degree-8 minimax polynomial on |z| <= 4.5 (z is clamped
// there, Phi to [0, 1]); absolute error below 2.2e-5, a hundred times under the 16-bit rounding of the result.
// Ten full-rate fused multiply-adds; erff(), or an erfc formula with a reciprocal and an exponential, cost two to
// four times that in issue slots (transcendentals run at quarter rate).
__device__ __forceinline__ float normal_cdf(float z) {
  const float zc = __builtin_amdgcn_fmed3f(z, -4.5f, 4.5f);
  const float u = zc * zc;
  float q = 3.805729969e-11f;
  q = fmaf(q, u, -4.002348328e-09f);
  q = fmaf(q, u, 1.846177390e-07f);
  q = fmaf(q, u, -4.959758083e-06f);
  q = fmaf(q, u, 8.727687015e-05f);
  q = fmaf(q, u, -1.076740563e-03f);
  q = fmaf(q, u, 9.729495093e-03f);
  q = fmaf(q, u, -6.624044322e-02f);
  q = fmaf(q, u, 3.988664908e-01f);
  return __builtin_amdgcn_fmed3f(fmaf(zc, q, 0.5f), 0.0f, 1.0f);
}
// exp(-z^2 / 2) / sqrt(2 pi)
__device__ __forceinline__ float normal_pdf(float z) { return 0.3989422804014327f * __expf(-0.5f * z * z); }
// CDF and density together, for the backward passes that need both: erfc through Abramowitz & Stegun 7.1.26
// (absolute error below 1.5e-7) shares its exponential with the density.
__device__ __forceinline__ float normal_cdf_pdf(float z, float* pdf) {
  const float x = fabsf(z) * 0.70710678118654752f;
  const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * x);  // v_rcp_f32, 1 ulp
  const float e = __expf(-x * x);
  const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
  const float q = 0.5f * poly * e;  // Phi(-|z|)
  *pdf = 0.3989422804014327f * e;
  return z >= 0.0f ? 1.0f - q : q;
}

// The same with the three-term form (Abramowitz & Stegun 7.1.25, absolute error of Phi and of Phi + z phi below 1.1e-5:
// half of what the forward's polynomial allows itself), fifteen instructions for both instead of eighteen; the scale
// 1/sqrt 2 of the argument is folded into the constants.
__device__ __forceinline__ float normal_cdf_pdf3(float z, float* pdf) {
  const float t = __builtin_amdgcn_rcpf(fmaf(0.33267252f, fabsf(z), 1.0f));  // 1 / (1 + 0.47047 |z| / sqrt 2); v_rcp_f32, 1 ulp
  const float e = __builtin_amdgcn_exp2f(z * z * -0.72134752f);              // exp(-z^2 / 2)
  const float q = t * (0.1740121f + t * (-0.0479399f + t * 0.3739278f)) * e;  // Phi(-|z|), the 1/2 folded into the coefficients
  *pdf = 0.3989422804014327f * e;
  return z >= 0.0f ? 1.0f - q : q;
}

// ---- activations (triton_helpers/ops.py:37-66 of the reference; gelu = erf form) ----
__device__ __forceinline__ float act_fwd(float z, int act) {
  switch (act) {
    case NF_ACT_RELU: return z < 0.0f ? 0.0f : z;
    case NF_ACT_SILU: return z * __builtin_amdgcn_rcpf(1.0f + __expf(-z));  // v_rcp_f32 (1 ulp) instead of a full division
    case NF_ACT_RELU2: return fmaxf(z, 0.0f) * z;
    case NF_ACT_GELU: return z * normal_cdf(z);
    default: return z;
  }
}
// derivative d act / d z
__device__ __forceinline__ float act_grad(float z, int act) {
  switch (act) {
    case NF_ACT_RELU: return z > 0.0f ? 1.0f : 0.0f;
    case NF_ACT_SILU: {
      const float s = __builtin_amdgcn_rcpf(1.0f + __expf(-z));
      return s * (z * (1.0f - s) + 1.0f);
    }
    case NF_ACT_RELU2: return z > 0.0f ? 2.0f * z : 0.0f;
    case NF_ACT_GELU: return normal_cdf(z) + z * normal_pdf(z);
    default: return 1.0f;
  }
}

// Runs body(std::integral_constant<int, ACT>) under one wave-uniform branch on `act`, so that everything inside
// sees the activation as a compile-time constant.  A switch evaluated per element gets flattened into
// "compute every activation, then select", which doubles the cost of a layer epilogue.
template <typename Body>
__device__ __forceinline__ void with_act(int act, Body&& body) {
  switch (act) {
    case NF_ACT_RELU: body(std::integral_constant<int, NF_ACT_RELU>{}); break;
    case NF_ACT_SILU: body(std::integral_constant<int, NF_ACT_SILU>{}); break;
    case NF_ACT_RELU2: body(std::integral_constant<int, NF_ACT_RELU2>{}); break;
    case NF_ACT_GELU: body(std::integral_constant<int, NF_ACT_GELU>{}); break;
    default: body(std::integral_constant<int, NF_ACT_NONE>{}); break;
  }
}

// h = act(z) packed to 16 bit.  RELU = true is the branch-free fast path; otherwise `act` selects (pass a constant,
// see with_act, wherever the call sits in a loop).
template <typename T, bool RELU>
__device__ __forceinline__ void act_pack(const f32x4_t z, int act, uint32_t& p01, uint32_t& p23) {
  if (RELU) {
    p01 = pack2<T>(fmaxf(z[0], 0.0f), fmaxf(z[1], 0.0f));
    p23 = pack2<T>(fmaxf(z[2], 0.0f), fmaxf(z[3], 0.0f));
  } else {
    p01 = pack2<T>(act_fwd(z[0], act), act_fwd(z[1], act));
    p23 = pack2<T>(act_fwd(z[2], act), act_fwd(z[3], act));
  }
}
// What the backward keeps per pre-activation: for ReLU the activation itself (its sign bit pattern
// tells the gate: h != 0  <=>  z > 0); otherwise act'(z) rounded to 16 bit.
template <typename T, bool RELU>
__device__ __forceinline__ void gate_pack(const f32x4_t z, int act, uint32_t h01, uint32_t h23, uint32_t& g01, uint32_t& g23) {
  if (RELU) {
    g01 = h01;
    g23 = h23;
  } else {
    g01 = pack2<T>(act_grad(z[0], act), act_grad(z[1], act));
    g23 = pack2<T>(act_grad(z[2], act), act_grad(z[3], act));
  }
}
// act() of the eight packed values of a fragment (a sub-network whose input is a pre-activation).
template <typename T>
__device__ __forceinline__ Frag act_frag(Frag f, int act) {
  with_act(act, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int q = 0; q < 4; ++q) f.w[q] = pack2<T>(act_fwd(unpack_lo<T>(f.w[q]), ACT), act_fwd(unpack_hi<T>(f.w[q]), ACT));
  });
  return f;
}
// v * act'(x) for the four values of a tile, x packed in (x01, x23).  ReLU selects rather than multiplies.
template <typename T>
__device__ __forceinline__ f32x4_t input_gate(f32x4_t v, uint32_t x01, uint32_t x23, int act) {
  const float x[4] = {unpack_lo<T>(x01), unpack_hi<T>(x01), unpack_lo<T>(x23), unpack_hi<T>(x23)};
  with_act(act, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = ACT == NF_ACT_RELU ? (x[r] > 0.0f ? v[r] : 0.0f) : v[r] * act_grad(x[r], ACT);
  });
  return v;
}

// dz = dh * act'(z) from the parked gate image, packed to 16 bit.
template <typename T, bool RELU>
__device__ __forceinline__ void gate_apply(const f32x4_t dh, uint32_t g01, uint32_t g23, uint32_t& p01, uint32_t& p23) {
  if (RELU) {
    p01 = pack2<T>((g01 & 0xffffu) ? dh[0] : 0.0f, (g01 >> 16) ? dh[1] : 0.0f);
    p23 = pack2<T>((g23 & 0xffffu) ? dh[2] : 0.0f, (g23 >> 16) ? dh[3] : 0.0f);
  } else {
    p01 = pack2<T>(dh[0] * unpack_lo<T>(g01), dh[1] * unpack_hi<T>(g01));
    p23 = pack2<T>(dh[2] * unpack_lo<T>(g23), dh[3] * unpack_hi<T>(g23));
  }
}

// ---- staging weights into LDS as A fragments ------------------------------------------
// dst: fragment array [MT][KC][64 lanes][8 elements]; element (mt, kc, lane(m,g), j) =
//   transposed ? W[kmap(kc,g,j)][mmap(mt,m)] : W[mmap(mt,m)][kmap(kc,g,j)]
// where W is [w_rows][w_cols] row-major, mmap(mt, m) = 16*mt + m, or wide_feature(mt, m) with WIDE_M; out-of-range
// entries are zero.
// NTHREADS > 0: the workgroup size is that compile-time constant, the loop is unrolled and all loads of a matrix
// are in flight together.
template <bool CHAIN, bool TRANSPOSED, int NTHREADS = 0, bool WIDE_M = false>
__device__ __forceinline__ void stage_weight_frags(uint16_t* dst, const uint16_t* w, int w_rows, int w_cols, int MT,
                                                   int KC, int tid, int nthreads) {
  // one unit = the 8 elements of one lane of one fragment; the 8 loads of a unit are independent
  const int units = MT * KC * 64;
  const bool vec_ok = !TRANSPOSED && (w_cols % 4 == 0) && ((uintptr_t)w % 8 == 0);
  auto stage_unit = [&](int u) {
    const int lane = u & 63;
    const int frag = u >> 6;
    const int kc = frag % KC, mt = frag / KC;
    const int m = WIDE_M ? wide_feature(mt, lane & 15) : 16 * mt + (lane & 15);
    const int g = lane >> 4;
    uint16_t v[8];
    if (vec_ok && m < w_rows) {
      // non-transposed rows are contiguous in k: two 8-byte pieces (chain order) or one 16-byte run (natural)
      const int k0 = CHAIN ? k_chain(kc, g, 0) : k_nat(kc, g, 0);
      const int k1 = CHAIN ? k_chain(kc, g, 4) : k_nat(kc, g, 4);
      uint2 lo = make_uint2(0u, 0u), hi = make_uint2(0u, 0u);
      if (k0 + 4 <= w_cols) lo = *reinterpret_cast<const uint2*>(w + (size_t)m * w_cols + k0);
      else
        for (int j = 0; j < 4; ++j)
          if (k0 + j < w_cols) reinterpret_cast<uint16_t*>(&lo)[j] = w[(size_t)m * w_cols + k0 + j];
      if (k1 + 4 <= w_cols) hi = *reinterpret_cast<const uint2*>(w + (size_t)m * w_cols + k1);
      else
        for (int j = 0; j < 4; ++j)
          if (k1 + j < w_cols) reinterpret_cast<uint16_t*>(&hi)[j] = w[(size_t)m * w_cols + k1 + j];
      *reinterpret_cast<uint4*>(dst + (size_t)u * 8) = make_uint4(lo.x, lo.y, hi.x, hi.y);
      return;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = CHAIN ? k_chain(kc, g, j) : k_nat(kc, g, j);
      const int r = TRANSPOSED ? k : m;
      const int c = TRANSPOSED ? m : k;
      v[j] = (r < w_rows && c < w_cols) ? w[(size_t)r * w_cols + c] : (uint16_t)0;
    }
    uint4 o;
    o.x = (uint32_t)v[0] | ((uint32_t)v[1] << 16);
    o.y = (uint32_t)v[2] | ((uint32_t)v[3] << 16);
    o.z = (uint32_t)v[4] | ((uint32_t)v[5] << 16);
    o.w = (uint32_t)v[6] | ((uint32_t)v[7] << 16);
    *reinterpret_cast<uint4*>(dst + (size_t)u * 8) = o;
  };
  if constexpr (NTHREADS > 0) {
#pragma unroll
    for (int u = tid; u < units; u += NTHREADS) stage_unit(u);
  } else {
    for (int u = tid; u < units; u += nthreads) stage_unit(u);
  }
}

__device__ __forceinline__ Frag lds_frag(const uint16_t* frags, int frag_index, int lane) {
  Frag f;
  f.u = *reinterpret_cast<const uint4*>(frags + ((size_t)frag_index * 64 + lane) * 8);
  return f;
}

// ---- global <-> row-per-lane fragments ---------------------------------------------------
// B fragment of K-chunk kc for 16 rows starting at row0: lane (n, g) gets features
// 32*kc + 8*g .. +7 of row row0 + n; zero beyond `rows` / `width`.
__device__ __forceinline__ Frag load_rows_frag(const uint16_t* base, int64_t stride, int64_t row0, int64_t rows,
                                               int width, int kc, int lane, bool vec_ok) {
  Frag f;
  f.u = make_uint4(0u, 0u, 0u, 0u);
  const int64_t r = row0 + (lane & 15);
  const int c0 = 32 * kc + 8 * (lane >> 4);
  if (r < rows && c0 < width) {
    const uint16_t* p = base + r * stride + c0;
    if (vec_ok && c0 + 8 <= width) {
      f.u = *reinterpret_cast<const uint4*>(p);
    } else {
      uint16_t tmp[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) tmp[j] = (c0 + j < width) ? p[j] : (uint16_t)0;
#pragma unroll
      for (int j = 0; j < 4; ++j) f.w[j] = (uint32_t)tmp[2 * j] | ((uint32_t)tmp[2 * j + 1] << 16);
    }
  }
  return f;
}

// Store accumulator tile mt (lane (n,g): features 16*mt + 4*g + r) of 16 rows as 16-bit values.
template <typename T>
__device__ __forceinline__ void store_rows_tile(uint16_t* base, int64_t stride, int64_t row0, int64_t rows, int width,
                                                int mt, int lane, f32x4_t v, bool vec_ok) {
  const int64_t r = row0 + (lane & 15);
  const int c0 = 16 * mt + 4 * (lane >> 4);
  if (r >= rows || c0 >= width) return;
  uint16_t* p = base + r * stride + c0;
  if (vec_ok && c0 + 4 <= width) {
    uint2 o;
    o.x = pack2<T>(v[0], v[1]);
    o.y = pack2<T>(v[2], v[3]);
    *reinterpret_cast<uint2*>(p) = o;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (c0 + i < width) p[i] = T::from_f32(v[i]);
  }
}

// The four stored values store_rows_tile() would overwrite, packed; zero beyond `rows` / `width`.
__device__ __forceinline__ uint2 load_rows_tile(const uint16_t* base, int64_t stride, int64_t row0, int64_t rows, int width,
                                               int mt, int lane, bool vec_ok) {
  const int64_t r = row0 + (lane & 15);
  const int c0 = 16 * mt + 4 * (lane >> 4);
  uint2 o = make_uint2(0u, 0u);
  if (r >= rows || c0 >= width) return o;
  const uint16_t* p = base + r * stride + c0;
  if (vec_ok && c0 + 4 <= width) return *reinterpret_cast<const uint2*>(p);
  uint16_t e[4] = {0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (c0 + i < width) e[i] = p[i];
  o.x = (uint32_t)e[0] | ((uint32_t)e[1] << 16);
  o.y = (uint32_t)e[2] | ((uint32_t)e[3] << 16);
  return o;
}

// ---- transposes and row sums for products that contract over the rows of a chunk -----------
// Transpose through the matrix core.  f0 / f1 are chain-order fragments of rows 0-15 / 16-31 of a chunk
// (lane (row, g): 8 features of K-chunk kc); e selects 16 of those 32 features (sel_frag()).  The product
// F * E has exactly one non-zero term per output, so it is exact; the result, packed back to 16 bit, is the
// operand of a product that contracts over the chunk's 32 rows: lane (feature, g) holds rows 4g .. 4g+3 and
// 16+4g .. 16+4g+3 of that feature.  Both operands of such a product use the same row order.
template <typename T>
__device__ __forceinline__ Frag transpose_tile(const Frag& f0, const Frag& f1, const Frag& e) {
  const f32x4_t z = {0.0f, 0.0f, 0.0f, 0.0f};
  const f32x4_t a = mfma16<T>(f0, e, z);
  const f32x4_t b = mfma16<T>(f1, e, z);
  Frag o;
  o.w[0] = pack2<T>(a[0], a[1]);
  o.w[1] = pack2<T>(a[2], a[3]);
  o.w[2] = pack2<T>(b[0], b[1]);
  o.w[3] = pack2<T>(b[2], b[3]);
  return o;
}
// Selector of features 16*half .. 16*half+15 of a chain-order K-chunk: B[k][n] = 1 where slot k holds feature
// 16*half + n, i.e. lane (n, g) with g == n / 4 carries a 1.0 in element 4*half + n % 4.
template <typename T>
__device__ __forceinline__ Frag sel_frag(int half, int lane) {
  const int n = lane & 15, g = lane >> 4;
  const uint32_t one = (pack2<T>(1.0f, 1.0f) & 0xffffu) << (16 * (n & 1));
  const uint32_t v = (g == (n >> 2)) ? one : 0u;
  const int d = 2 * half + ((n & 3) >> 1);
  Frag e;
#pragma unroll
  for (int i = 0; i < 4; ++i) e.w[i] = (i == d) ? v : 0u;
  return e;
}

// Transpose through LDS with gfx950's transposing reads.  A wave parks the row-per-lane fragments of a 32-row chunk as a
// row-major panel panel[row][feature] (TR_STRIDE dwords per row: 64 features + 2, so the 16 rows a store instruction
// touches fall on 16 different bank pairs and the rows r, r+4, r+8, r+12 of one read on disjoint 8-bank windows), then
// reads, for a tile of 16 features, lane (i, g) <- feature 16*tile + i of the rows g + 4k (k = 0..3) and 16 + g + 4k: the
// operand of a product that contracts over the chunk's 32 rows.  Both operands of such a product come from here, so
// they share the row order.  ds_read_b64_tr_b16: within 16 lanes, lane p supplies the address of 4 consecutive 16-bit
// values M[p][0..3]; lane i receives M[4k + i / 4][i % 4], k = 0..3.  LDS operations of one wave complete in order, so
// a wave that parks and reads its own panel needs no barrier.
constexpr int TR_STRIDE = 34;
constexpr int TR_PANEL_DWORDS = 32 * TR_STRIDE;
// fragment f = K-chunk kc (chain order) of row tile nt (rows 16*nt .. 16*nt+15)
template <bool BOTH_HALVES = true>
__device__ __forceinline__ void park_frag_rows(uint32_t* panel, const Frag& f, int nt, int kc, int lane) {
  uint32_t* p = panel + (16 * nt + (lane & 15)) * TR_STRIDE + 16 * kc + 2 * (lane >> 4);
  *reinterpret_cast<uint2*>(p) = make_uint2(f.w[0], f.w[1]);                       // features 32*kc + 4g .. +3
  if (BOTH_HALVES) *reinterpret_cast<uint2*>(p + 8) = make_uint2(f.w[2], f.w[3]);  // features 32*kc + 16 + 4g .. +3
}
typedef short tr_v4i16 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ Frag tr_operand(const uint32_t* panel, int tile, int lane) {
  const int i = lane & 15, g = lane >> 4;
  const uint32_t* p = panel + (g + 4 * (i >> 2)) * TR_STRIDE + 8 * tile + 2 * (i & 3);
  typedef tr_v4i16 __attribute__((address_space(3))) * lds_ptr;
  const tr_v4i16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p);
  const tr_v4i16 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 16 * TR_STRIDE));
  Frag f;
  const uint2 a = __builtin_bit_cast(uint2, lo), b = __builtin_bit_cast(uint2, hi);
  f.w[0] = a.x;
  f.w[1] = a.y;
  f.w[2] = b.x;
  f.w[3] = b.y;
  return f;
}

// acc + lo + hi of a packed 16-bit pair (one v_dot2 instruction)
template <typename T>
__device__ __forceinline__ float dot2_ones(uint32_t p, float acc);
template <>
__device__ __forceinline__ float dot2_ones<BF16>(uint32_t p, float acc) {
  const bf16x2_t one = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p), one, acc, false);
}
template <>
__device__ __forceinline__ float dot2_ones<F16>(uint32_t p, float acc) {
  const f16x2_t one = {(_Float16)1.0f, (_Float16)1.0f};
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, p), one, acc, false);
}

inline bool vec_load_ok(const void* p, int64_t stride_elems, int width) {
  return ((uintptr_t)p % 16 == 0) && (stride_elems % 8 == 0) && (width % 8 == 0);
}
inline bool vec_store_ok(const void* p, int64_t stride_elems, int width) {
  return ((uintptr_t)p % 8 == 0) && (stride_elems % 4 == 0) && (width % 4 == 0);
}

}  // namespace nf
