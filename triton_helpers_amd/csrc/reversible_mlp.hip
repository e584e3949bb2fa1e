// Reversible (additive-coupling) fused MLP for gfx950, 16-bit storage, MFMA 16x16x32.
//
//   block k:  y1 = x1 + F_k(x2),  y2 = x2 + G_k(y1),   F/G(u) = act(u W1^T + b1) W2^T + b2
//
// Forward: one launch runs up to FWD_GROUP coupling blocks with all their weights resident
// in LDS; the two halves of the residual stream stay in float32 registers between blocks.
// Backward: one launch walks the coupling blocks, last block first, a wave keeping its rows.  For
// each block it takes the block's OUTPUT (y, dy), rebuilds the block's input in-kernel
// (x2 = y2 - G(y1), x1 = y1 - F(x2)) while it back-propagates, and writes (x, dx), which it reads
// back in place for the block below after restaging that block's weights.  No activation
// of the forward pass is ever stored.  The four weight gradients of a block accumulate in
// float32 registers over the wave's whole row loop (the fourth of a 64-wide block in LDS); their
// operands (rows along K) are matrix-core transposes of the row-per-lane fragments, so LDS otherwise
// only holds weights.  The backward numbers the stream's features in "wide order" (wide_feature()
// in mlp_tile.h), which lets a lane reach the eight features of two accumulator tiles with one
// 16-byte access; the staged weights and the flushed gradients absorb the permutation.
//
// There is no counterpart in the reference; the layer math is that of its fused MLP
// (triton_helpers/layers/fully_fused_mlp/kernel.py:17-74).
#include "mlp_tile.h"

namespace nf {

constexpr int RFRAG = 64 * 8;
constexpr int FWD_GROUP = 4;   // coupling blocks per forward launch (LDS: 32 KiB of weights per block at H = 64)

struct RevArgs {
  const uint16_t* in;   // fwd: x ; bwd: y of this block
  int64_t in_stride;
  uint16_t* out;        // fwd: y ; bwd: reconstructed x
  int64_t out_stride;
  const uint16_t* dy;
  int64_t dy_stride;
  uint16_t* dx;
  int64_t dx_stride;
  const uint16_t *w1, *b1, *w2, *b2;  // first coupling of this launch
  float *dw1, *db1, *dw2, *db2;       // first coupling of this launch (backward)
  int64_t rows;
  int half, nblocks, act;
  int vec_in, vec_out, vec_dy, vec_dx;
  int wide_ok;  // backward: every tensor allows 16-byte accesses to its rows
};

// accumulator-layout load: lane (n,g) gets features 16*mt + 4*g + r of row row0 + n as two packed dwords
// (WIDE: features wide_feature(mt, 4*g + r) instead)
template <bool WIDE = false>
__device__ __forceinline__ uint2 load_tile_packed(const uint16_t* base, int64_t stride, int64_t row0, int64_t rows, int col0,
                                                  int width, int mt, int lane, bool vec_ok) {
  uint2 v = make_uint2(0u, 0u);
  const int64_t r = row0 + (lane & 15);
  const int c = WIDE ? wide_feature(mt, 4 * (lane >> 4)) : 16 * mt + 4 * (lane >> 4);
  if (r < rows && c < width) {
    const uint16_t* p = base + r * stride + col0 + c;
    if (vec_ok && c + 4 <= width) {
      v = *reinterpret_cast<const uint2*>(p);
    } else {
      uint16_t t[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) t[i] = (c + i < width) ? p[i] : (uint16_t)0;
      v.x = (uint32_t)t[0] | ((uint32_t)t[1] << 16);
      v.y = (uint32_t)t[2] | ((uint32_t)t[3] << 16);
    }
  }
  return v;
}
template <bool WIDE = false>
__device__ __forceinline__ void store_tile_packed(uint16_t* base, int64_t stride, int64_t row0, int64_t rows, int col0,
                                                  int width, int mt, int lane, uint2 v, bool vec_ok) {
  const int64_t r = row0 + (lane & 15);
  const int c = WIDE ? wide_feature(mt, 4 * (lane >> 4)) : 16 * mt + 4 * (lane >> 4);
  if (r >= rows || c >= width) return;
  uint16_t* p = base + r * stride + col0 + c;
  if (vec_ok && c + 4 <= width) {
    *reinterpret_cast<uint2*>(p) = v;
  } else {
    const uint16_t t[4] = {(uint16_t)(v.x & 0xffffu), (uint16_t)(v.x >> 16), (uint16_t)(v.y & 0xffffu), (uint16_t)(v.y >> 16)};
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (c + i < width) p[i] = t[i];
  }
}

// The same tiles when the caller knows that H is the padded width, that every row allows 8-byte accesses and that
// no chunk is ragged: one address per (tensor, row tile), the column part is an immediate offset.
template <bool FAST>
__device__ __forceinline__ uint2 ld_tile(const uint16_t* base, int64_t stride, int64_t row0, int64_t rows, int col0,
                                         int width, int mt, int lane, bool vec_ok) {
  if (FAST) return *reinterpret_cast<const uint2*>(base + (row0 + (lane & 15)) * stride + 4 * (lane >> 4) + col0 + 16 * mt);
  return load_tile_packed<false>(base, stride, row0, rows, col0, width, mt, lane, vec_ok);
}
template <bool FAST>
__device__ __forceinline__ void st_tile(uint16_t* base, int64_t stride, int64_t row0, int64_t rows, int col0, int width,
                                        int mt, int lane, uint2 v, bool vec_ok) {
  if (FAST) {
    *reinterpret_cast<uint2*>(base + (row0 + (lane & 15)) * stride + 4 * (lane >> 4) + col0 + 16 * mt) = v;
    return;
  }
  store_tile_packed<false>(base, stride, row0, rows, col0, width, mt, lane, v, vec_ok);
}

// Tiles 2p and 2p + 1 of a row tile in wide order (wide_feature()): lane (n, g) holds features 32p + 8g .. + 7 of row
// row0 + n, one 16-byte access.  Only for full-width, 16-byte aligned, unragged tensors.
__device__ __forceinline__ void ld_tile_pair(const uint16_t* base, int64_t stride, int64_t row0, int col0, int p, int lane,
                                             uint2& t0, uint2& t1) {
  const uint4 v = *reinterpret_cast<const uint4*>(base + (row0 + (lane & 15)) * stride + col0 + 32 * p + 8 * (lane >> 4));
  t0 = make_uint2(v.x, v.y);
  t1 = make_uint2(v.z, v.w);
}
__device__ __forceinline__ void st_tile_pair(uint16_t* base, int64_t stride, int64_t row0, int col0, int p, int lane, uint2 t0,
                                             uint2 t1) {
  *reinterpret_cast<uint4*>(base + (row0 + (lane & 15)) * stride + col0 + 32 * p + 8 * (lane >> 4)) = make_uint4(t0.x, t0.y, t1.x, t1.y);
}

template <typename T>
__device__ __forceinline__ f32x4_t unpack4(uint2 v) {
  f32x4_t o = {unpack_lo<T>(v.x), unpack_hi<T>(v.x), unpack_lo<T>(v.y), unpack_hi<T>(v.y)};
  return o;
}
template <typename T>
__device__ __forceinline__ uint2 pack4(f32x4_t v) {
  return make_uint2(pack2<T>(v[0], v[1]), pack2<T>(v[2], v[3]));
}

// packed accumulator-layout tiles P[nt][mt] -> B fragments (chain order) F[nt][kc]
template <int MT>
__device__ __forceinline__ void tiles_to_frags(const uint2 (&p)[2][4], Frag (&f)[2][2]) {
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      f[nt][mt >> 1].w[2 * (mt & 1)] = p[nt][mt].x;
      f[nt][mt >> 1].w[2 * (mt & 1) + 1] = p[nt][mt].y;
    }
}

// K chunks outermost: the two products into one accumulator tile are MT * 2 instructions apart.
template <typename T, int MT, int KC>
__device__ __forceinline__ void rev_layer(f32x4_t (&acc)[2][4], const Frag (&in)[2][2], const uint16_t* frags, const float* bias,
                                          int lane) {
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    f32x4_t b4 = {0.0f, 0.0f, 0.0f, 0.0f};
    if (bias != nullptr) b4 = *reinterpret_cast<const f32x4_t*>(bias + 16 * mt + 4 * (lane >> 4));
    acc[0][mt] = b4;
    acc[1][mt] = b4;
  }
#pragma unroll
  for (int kc = 0; kc < KC; ++kc)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const Frag a = lds_frag(frags, mt * KC + kc, lane);
      acc[0][mt] = mfma16<T>(a, in[0][kc], acc[0][mt]);
      acc[1][mt] = mfma16<T>(a, in[1][kc], acc[1][mt]);
    }
}

// WIDE: position 16*mt + m of the staged row holds the bias of feature wide_feature(mt, m)
template <typename T, bool WIDE = false>
__device__ __forceinline__ void stage_bias_row(float* dst, const uint16_t* b, int n_valid, int n_pad, int tid, int nthreads) {
  for (int i = tid; i < n_pad; i += nthreads) {
    const int f = WIDE ? wide_feature(i >> 4, i & 15) : i;
    dst[i] = (b != nullptr && f < n_valid) ? T::to_f32(b[f]) : 0.0f;
  }
}

// ---------------------------------------------------------------------------------------
// Forward: up to FWD_GROUP blocks per launch
// ---------------------------------------------------------------------------------------
// ACT >= 0 fixes the activation at compile time (no per-element selection); -1 reads it from the arguments.
template <typename T, int HP, int ACT, bool FAST>
__global__ __launch_bounds__(768) void rev_fwd_k(RevArgs a) {
  constexpr int MT = HP / 16, KC = HP / 32, LAYER = MT * KC * RFRAG;
  const int act = ACT >= 0 ? ACT : a.act;
  const int nwaves = (int)(blockDim.x >> 6);
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, nthreads = blockDim.x, lane = tid & 63, wave = tid >> 6;
  uint16_t* frags = reinterpret_cast<uint16_t*>(smem);  // [nblocks][F.w1, F.w2, G.w1, G.w2][LAYER]
  float* bias = reinterpret_cast<float*>(frags + (size_t)a.nblocks * 4 * LAYER);  // [nblocks][4][HP]
  const int H = FAST ? HP : a.half;
  for (int k = 0; k < a.nblocks; ++k)
    for (int s = 0; s < 2; ++s) {
      const size_t sub = (size_t)(2 * k + s);
      stage_weight_frags<true, false>(frags + ((size_t)k * 4 + 2 * s) * LAYER, a.w1 + sub * H * H, H, H, MT, KC, tid, nthreads);
      stage_weight_frags<true, false>(frags + ((size_t)k * 4 + 2 * s + 1) * LAYER, a.w2 + sub * H * H, H, H, MT, KC, tid, nthreads);
      stage_bias_row<T>(bias + ((size_t)k * 4 + 2 * s) * HP, a.b1 ? a.b1 + sub * H : nullptr, H, HP, tid, nthreads);
      stage_bias_row<T>(bias + ((size_t)k * 4 + 2 * s + 1) * HP, a.b2 ? a.b2 + sub * H : nullptr, H, HP, tid, nthreads);
    }
  __syncthreads();

  const int64_t n_chunks = (a.rows + 31) / 32;
  for (int64_t chunk = (int64_t)blockIdx.x * nwaves + wave; chunk < n_chunks; chunk += (int64_t)gridDim.x * nwaves) {
    const int64_t row0 = chunk * 32;
    f32x4_t s1[2][4], s2[2][4];  // the two halves of the residual stream, float32
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        s1[nt][mt] = unpack4<T>(ld_tile<FAST>(a.in, a.in_stride, row0 + 16 * nt, a.rows, 0, H, mt, lane, a.vec_in));
        s2[nt][mt] = unpack4<T>(ld_tile<FAST>(a.in, a.in_stride, row0 + 16 * nt, a.rows, H, H, mt, lane, a.vec_in));
      }
    for (int k = 0; k < a.nblocks; ++k) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        // s == 0: s1 += F(s2) ; s == 1: s2 += G(s1)
        f32x4_t(&src)[2][4] = s == 0 ? s2 : s1;
        f32x4_t(&dst)[2][4] = s == 0 ? s1 : s2;
        const uint16_t* fw1 = frags + ((size_t)k * 4 + 2 * s) * LAYER;
        const float* bb1 = bias + ((size_t)k * 4 + 2 * s) * HP;
        uint2 p[2][4];
        Frag u[2][2], t[2][2];
        f32x4_t acc[2][4];
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) p[nt][mt] = pack4<T>(src[nt][mt]);
        tiles_to_frags<MT>(p, u);
        rev_layer<T, MT, KC>(acc, u, fw1, bb1, lane);
        with_act(act, [&](auto act_c) {
          constexpr int A = decltype(act_c)::value;
#pragma unroll
          for (int nt = 0; nt < 2; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              f32x4_t z = acc[nt][mt];
#pragma unroll
              for (int r = 0; r < 4; ++r) z[r] = act_fwd(z[r], A);
              p[nt][mt] = pack4<T>(z);
            }
        });
        tiles_to_frags<MT>(p, t);
        rev_layer<T, MT, KC>(acc, t, fw1 + LAYER, bb1 + HP, lane);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) dst[nt][mt] += acc[nt][mt];
      }
    }
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        st_tile<FAST>(a.out, a.out_stride, row0 + 16 * nt, a.rows, 0, H, mt, lane, pack4<T>(s1[nt][mt]), a.vec_out);
        st_tile<FAST>(a.out, a.out_stride, row0 + 16 * nt, a.rows, H, H, mt, lane, pack4<T>(s2[nt][mt]), a.vec_out);
      }
  }
}

// ---------------------------------------------------------------------------------------
// Backward of one coupling block
// ---------------------------------------------------------------------------------------
// Activation and its derivative from one pre-activation (GELU shares the exponential between the two).
template <int ACT>
__device__ __forceinline__ void act_both(float z, float& h, float& g) {
  if (ACT == NF_ACT_GELU) {
    float pdf;
    const float cdf = normal_cdf_pdf3(z, &pdf);
    h = z * cdf;
    g = cdf + z * pdf;
  } else if (ACT == NF_ACT_RELU) {
    h = fmaxf(z, 0.0f);
    g = z > 0.0f ? 1.0f : 0.0f;
  } else {
    h = act_fwd(z, ACT);
    g = act_grad(z, ACT);
  }
}

// Back-propagate through one sub-MLP  out = in_other + S(u):
//   given u (packed tiles), the incoming gradient d (packed tiles) w.r.t. S's output, computes
//   s_out = S(u) (float32, returned in `sout`), accumulates dW1, dW2 (and db), and returns du = W1^T dz.
// The operands of the weight-gradient products (rows along K) come from matrix-core transposes of the
// row-per-lane fragments; nothing goes through LDS but the weights.
// dw2_lds != nullptr: this wave's dW2 accumulator tiles live there ([MT*MT][64 lanes] float4) instead of dw2.
template <typename T, int MT, int KC, int ACT>
__device__ __forceinline__ void sub_backward(const uint2 (&u)[2][4], const uint2 (&d)[2][4], f32x4_t (&sout)[2][4],
                                             f32x4_t (&du)[2][4], f32x4_t (&dw1)[4][4], f32x4_t (&dw2)[4][4], f32x4_t* dw2_lds,
                                             float (&db1)[4], float (&db2)[4], const uint16_t* fw1, const uint16_t* fw2,
                                             const uint16_t* tw1, const uint16_t* tw2, const float* b1, const float* b2,
                                             const Frag (&sel)[2], int act, int lane) {
  Frag uf[2][2], tf[2][2], df[2][2], dzf[2][2];
  uint2 tp[2][4], gp[2][4];
  f32x4_t acc[2][4];
  tiles_to_frags<MT>(u, uf);
  tiles_to_frags<MT>(d, df);
  // recompute hidden activation t = act(W1 u + b1) and act'(z)
  rev_layer<T, MT, KC>(acc, uf, fw1, b1, lane);
  with_act(act, [&](auto act_c) {
    constexpr int A = decltype(act_c)::value;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        f32x4_t h, g;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float hv, gv;
          act_both<A>(acc[nt][mt][r], hv, gv);
          h[r] = hv;
          g[r] = gv;
        }
        tp[nt][mt] = pack4<T>(h);
        gp[nt][mt] = pack4<T>(g);
      }
  });
  tiles_to_frags<MT>(tp, tf);
  // S(u) = W2 t + b2
  rev_layer<T, MT, KC>(sout, tf, fw2, b2, lane);
  // dW2 += d^T t, db2 += sum d
  {
    Frag tb[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) tb[j] = transpose_tile<T>(tf[0][j >> 1], tf[1][j >> 1], sel[j & 1]);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      if (dw2_lds != nullptr) {
        // the row's accumulator tiles are asked for before the transpose that their products wait for anyway
        f32x4_t c[MT];
#pragma unroll
        for (int j = 0; j < MT; ++j) c[j] = dw2_lds[(i * MT + j) * 64 + lane];
        const Frag da = transpose_tile<T>(df[0][i >> 1], df[1][i >> 1], sel[i & 1]);
#pragma unroll
        for (int j = 0; j < MT; ++j) c[j] = mfma16<T>(da, tb[j], c[j]);
#pragma unroll
        for (int j = 0; j < MT; ++j) dw2_lds[(i * MT + j) * 64 + lane] = c[j];
#pragma unroll
        for (int q = 0; q < 4; ++q) db2[i] = dot2_ones<T>(da.w[q], db2[i]);
        continue;
      }
      const Frag da = transpose_tile<T>(df[0][i >> 1], df[1][i >> 1], sel[i & 1]);
      {
#pragma unroll
        for (int j = 0; j < MT; ++j) dw2[i][j] = mfma16<T>(da, tb[j], dw2[i][j]);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) db2[i] = dot2_ones<T>(da.w[q], db2[i]);
    }
  }
  // dt = W2^T d ; dz = dt * act'(z)
  rev_layer<T, MT, KC>(acc, df, tw2, nullptr, lane);
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const f32x4_t g = unpack4<T>(gp[nt][mt]);
      f32x4_t dz;
#pragma unroll
      for (int r = 0; r < 4; ++r) dz[r] = acc[nt][mt][r] * g[r];
      tp[nt][mt] = pack4<T>(dz);
    }
  tiles_to_frags<MT>(tp, dzf);
  // dW1 += dz^T u, db1 += sum dz
  {
    Frag ub[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) ub[j] = transpose_tile<T>(uf[0][j >> 1], uf[1][j >> 1], sel[j & 1]);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const Frag da = transpose_tile<T>(dzf[0][i >> 1], dzf[1][i >> 1], sel[i & 1]);
#pragma unroll
      for (int j = 0; j < MT; ++j) dw1[i][j] = mfma16<T>(da, ub[j], dw1[i][j]);
#pragma unroll
      for (int q = 0; q < 4; ++q) db1[i] = dot2_ones<T>(da.w[q], db1[i]);
    }
  }
  // du = W1^T dz
  rev_layer<T, MT, KC>(du, dzf, tw1, nullptr, lane);
}

// Bias gradient of feature 16*mt + n: the four lane groups hold partial sums over disjoint rows.
// WIDE: the tile's features are in wide order (wide_feature())
template <bool WIDE = false>
__device__ __forceinline__ void flush_db_rev(float* db, int dim, int mt, int lane, float v) {
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  const int f = WIDE ? wide_feature(mt, lane & 15) : 16 * mt + lane;
  if (db != nullptr && lane < 16 && f < dim) unsafeAtomicAdd(db + f, v);
}

// WIDE_ROWS / WIDE_COLS: the tile's rows (mt) / columns (nt) are features in wide order
template <bool WIDE_ROWS = false, bool WIDE_COLS = false>
__device__ __forceinline__ void flush_tile(float* dw, int dim, int mt, int nt, int lane, f32x4_t v) {
  const int c = WIDE_COLS ? wide_feature(nt, lane & 15) : 16 * nt + (lane & 15);
  const int r0 = WIDE_ROWS ? wide_feature(mt, 4 * (lane >> 4)) : 16 * mt + 4 * (lane >> 4);
  if (c >= dim) return;
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (r0 + r < dim) unsafeAtomicAdd(dw + (size_t)(r0 + r) * dim + c, v[r]);
}

template <typename T, int HP, int ACT, bool FAST>
__global__ __launch_bounds__(256) void rev_bwd_block_k(RevArgs a) {
  constexpr int MT = HP / 16, KC = HP / 32, LAYER = MT * KC * RFRAG;
  // The backward keeps the stream's features in wide order: the unchecked variant then reaches its rows with 16-byte
  // accesses, half as many of them (a tile access has one lane per row and line, so the vector memory pipeline sees every
  // lane as an access of its own); the checked variant uses the same order, so both do the same arithmetic.
  constexpr bool WIDE = true;
  const int act = ACT >= 0 ? ACT : a.act;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, nthreads = blockDim.x, lane = tid & 63, wave = tid >> 6;
  const int H = FAST ? HP : a.half;
  // weights: forward-form [F.w1, F.w2, G.w1, G.w2], transposed-form the same order
  uint16_t* fw = reinterpret_cast<uint16_t*>(smem);
  uint16_t* tw = fw + 4 * LAYER;
  float* bias = reinterpret_cast<float*>(tw + 4 * LAYER);  // [4][HP]
  // Four 64x64 float32 accumulators would fill the whole accumulation register file and leave none for the
  // layer products: at HP = 64 the fourth (G's second layer) lives in LDS, 16 KiB per wave.
  constexpr bool G2_LDS = HP > 32;
  f32x4_t* g2acc = G2_LDS ? reinterpret_cast<f32x4_t*>(bias + 4 * HP) + (size_t)wave * MT * MT * 64 : nullptr;
  const Frag sel[2] = {sel_frag<T>(0, lane), sel_frag<T>(1, lane)};
  const f32x4_t zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
  const int64_t n_chunks = (a.rows + 31) / 32;

  // The couplings of the launch, last first.  A wave owns the same rows in every coupling, so it reads (x, dx) of the
  // coupling above from where it wrote them itself and no workgroup ever waits for another; the weight-gradient
  // atomics of one coupling drain while the next is being computed.
  // (Only the variant without per-tile checks loops; the general one is launched once per coupling.)
  for (int kb = FAST ? a.nblocks - 1 : 0; kb >= 0; --kb) {
  const bool top = FAST ? kb == a.nblocks - 1 : true;
  const uint16_t* in_p = top ? a.in : a.out;
  const int64_t in_s = top ? a.in_stride : a.out_stride;
  const bool in_v = top ? a.vec_in : a.vec_out;
  const uint16_t* dy_p = top ? a.dy : a.dx;
  const int64_t dy_s = top ? a.dy_stride : a.dx_stride;
  const bool dy_v = top ? a.vec_dy : a.vec_dx;
  const uint16_t* w1 = a.w1 + (size_t)2 * kb * H * H;
  const uint16_t* w2 = a.w2 + (size_t)2 * kb * H * H;
  const uint16_t* b1 = a.b1 ? a.b1 + (size_t)2 * kb * H : nullptr;
  const uint16_t* b2 = a.b2 ? a.b2 + (size_t)2 * kb * H : nullptr;
  if (G2_LDS)
    for (int i = lane; i < MT * MT * 64; i += 64) g2acc[i] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  for (int s = 0; s < 2; ++s) {
    // WIDE: the stream's features are contracted in natural order and produced in wide order (the hidden ones as ever)
    stage_weight_frags<!WIDE, false>(fw + (2 * s) * LAYER, w1 + (size_t)s * H * H, H, H, MT, KC, tid, nthreads);
    stage_weight_frags<true, false, 0, WIDE>(fw + (2 * s + 1) * LAYER, w2 + (size_t)s * H * H, H, H, MT, KC, tid, nthreads);
    stage_weight_frags<true, true, 0, WIDE>(tw + (2 * s) * LAYER, w1 + (size_t)s * H * H, H, H, MT, KC, tid, nthreads);
    stage_weight_frags<!WIDE, true>(tw + (2 * s + 1) * LAYER, w2 + (size_t)s * H * H, H, H, MT, KC, tid, nthreads);
    stage_bias_row<T>(bias + (2 * s) * HP, b1 ? b1 + (size_t)s * H : nullptr, H, HP, tid, nthreads);
    stage_bias_row<T, WIDE>(bias + (2 * s + 1) * HP, b2 ? b2 + (size_t)s * H : nullptr, H, HP, tid, nthreads);
  }
  __syncthreads();

  f32x4_t dwF1[4][4], dwF2[4][4], dwG1[4][4], dwG2[4][4];
  // lane (feature, g) of tile i: partial bias gradient of feature 16*i + n over the rows of lane group g
  float dbF1[4] = {0.0f, 0.0f, 0.0f, 0.0f}, dbF2[4] = {0.0f, 0.0f, 0.0f, 0.0f}, dbG1[4] = {0.0f, 0.0f, 0.0f, 0.0f},
        dbG2[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) dwF1[i][j] = dwF2[i][j] = dwG1[i][j] = dwG2[i][j] = zero4;

  for (int64_t chunk = (int64_t)blockIdx.x * 4 + wave; chunk < n_chunks; chunk += (int64_t)gridDim.x * 4) {
    const int64_t row0 = chunk * 32;
    // The halves of y and dy that a sub-MLP's residual adds need are requested before that sub-MLP runs, so their
    // latency hides behind its products; nothing is held across both sub-MLPs (registers are the scarce resource).
    uint2 x2[2][4], d1[2][4];
    f32x4_t sout[2][4], du[2][4];
    {
      uint2 y1[2][4], d2[2][4], y2[2][4], dy1[2][4];
      if constexpr (FAST) {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int p = 0; p < MT / 2; ++p) {
            ld_tile_pair(in_p, in_s, row0 + 16 * nt, 0, p, lane, y1[nt][2 * p], y1[nt][2 * p + 1]);
            ld_tile_pair(dy_p, dy_s, row0 + 16 * nt, H, p, lane, d2[nt][2 * p], d2[nt][2 * p + 1]);
          }
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int p = 0; p < MT / 2; ++p) {
            ld_tile_pair(in_p, in_s, row0 + 16 * nt, H, p, lane, y2[nt][2 * p], y2[nt][2 * p + 1]);
            ld_tile_pair(dy_p, dy_s, row0 + 16 * nt, 0, p, lane, dy1[nt][2 * p], dy1[nt][2 * p + 1]);
          }
      } else {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          y1[nt][mt] = load_tile_packed<WIDE>(in_p, in_s, row0 + 16 * nt, a.rows, 0, H, mt, lane, in_v);
          d2[nt][mt] = load_tile_packed<WIDE>(dy_p, dy_s, row0 + 16 * nt, a.rows, H, H, mt, lane, dy_v);
        }
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          y2[nt][mt] = load_tile_packed<WIDE>(in_p, in_s, row0 + 16 * nt, a.rows, H, H, mt, lane, in_v);
          dy1[nt][mt] = load_tile_packed<WIDE>(dy_p, dy_s, row0 + 16 * nt, a.rows, 0, H, mt, lane, dy_v);
        }
      }
      // ---- G:  y2 = x2 + G(y1)  =>  x2 = y2 - G(y1),  dy1 += (dG/dy1)^T dy2
      sub_backward<T, MT, KC, ACT>(y1, d2, sout, du, dwG1, dwG2, g2acc, dbG1, dbG2, fw + 2 * LAYER, fw + 3 * LAYER,
                                   tw + 2 * LAYER, tw + 3 * LAYER, bias + 2 * HP, bias + 3 * HP, sel, act, lane);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          x2[nt][mt] = pack4<T>(unpack4<T>(y2[nt][mt]) - sout[nt][mt]);
          d1[nt][mt] = pack4<T>(unpack4<T>(dy1[nt][mt]) + du[nt][mt]);
        }
    }
    {
      // the other halves again (L2 hits), in flight during F
      uint2 y1[2][4], d2[2][4];
      if constexpr (FAST) {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int p = 0; p < MT / 2; ++p) {
            ld_tile_pair(in_p, in_s, row0 + 16 * nt, 0, p, lane, y1[nt][2 * p], y1[nt][2 * p + 1]);
            ld_tile_pair(dy_p, dy_s, row0 + 16 * nt, H, p, lane, d2[nt][2 * p], d2[nt][2 * p + 1]);
          }
      } else {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          y1[nt][mt] = load_tile_packed<WIDE>(in_p, in_s, row0 + 16 * nt, a.rows, 0, H, mt, lane, in_v);
          d2[nt][mt] = load_tile_packed<WIDE>(dy_p, dy_s, row0 + 16 * nt, a.rows, H, H, mt, lane, dy_v);
        }
      }
      // ---- F:  y1 = x1 + F(x2)  =>  x1 = y1 - F(x2),  dx2 = dy2 + (dF/dx2)^T dy1
      sub_backward<T, MT, KC, ACT>(x2, d1, sout, du, dwF1, dwF2, nullptr, dbF1, dbF2, fw, fw + LAYER, tw, tw + LAYER, bias,
                                   bias + HP, sel, act, lane);
      if constexpr (FAST) {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int p = 0; p < MT / 2; ++p) {
            uint2 x1[2], dx2[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              x1[e] = pack4<T>(unpack4<T>(y1[nt][2 * p + e]) - sout[nt][2 * p + e]);
              dx2[e] = pack4<T>(unpack4<T>(d2[nt][2 * p + e]) + du[nt][2 * p + e]);
            }
            st_tile_pair(a.out, a.out_stride, row0 + 16 * nt, 0, p, lane, x1[0], x1[1]);
            st_tile_pair(a.out, a.out_stride, row0 + 16 * nt, H, p, lane, x2[nt][2 * p], x2[nt][2 * p + 1]);
            st_tile_pair(a.dx, a.dx_stride, row0 + 16 * nt, 0, p, lane, d1[nt][2 * p], d1[nt][2 * p + 1]);
            st_tile_pair(a.dx, a.dx_stride, row0 + 16 * nt, H, p, lane, dx2[0], dx2[1]);
          }
      } else {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const uint2 x1 = pack4<T>(unpack4<T>(y1[nt][mt]) - sout[nt][mt]);
          const uint2 dx2 = pack4<T>(unpack4<T>(d2[nt][mt]) + du[nt][mt]);
          store_tile_packed<WIDE>(a.out, a.out_stride, row0 + 16 * nt, a.rows, 0, H, mt, lane, x1, a.vec_out);
          store_tile_packed<WIDE>(a.out, a.out_stride, row0 + 16 * nt, a.rows, H, H, mt, lane, x2[nt][mt], a.vec_out);
          store_tile_packed<WIDE>(a.dx, a.dx_stride, row0 + 16 * nt, a.rows, 0, H, mt, lane, d1[nt][mt], a.vec_dx);
          store_tile_packed<WIDE>(a.dx, a.dx_stride, row0 + 16 * nt, a.rows, H, H, mt, lane, dx2, a.vec_dx);
        }
      }
    }
  }

  // ---- weight gradients: summed over the four waves through LDS (the weight fragments are dead by now), then one
  // pass of 64-byte coalesced atomics per workgroup ----
  __syncthreads();
  constexpr int NREG = G2_LDS ? 3 : 4;  // accumulators that live in registers
  f32x4_t* red = reinterpret_cast<f32x4_t*>(smem) + lane;
  float* redb = reinterpret_cast<float*>(smem) + (size_t)NREG * MT * MT * 256 + lane;
  for (int w = 1; w < 4; ++w) {
    if (wave == w) {
      int t = 0, u = 0;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          red[64 * (t++)] = dwF1[i][j];
          red[64 * (t++)] = dwF2[i][j];
          red[64 * (t++)] = dwG1[i][j];
          if (!G2_LDS) red[64 * (t++)] = dwG2[i][j];
        }
        redb[64 * (u++)] = dbF1[i];
        redb[64 * (u++)] = dbF2[i];
        redb[64 * (u++)] = dbG1[i];
        redb[64 * (u++)] = dbG2[i];
      }
    }
    __syncthreads();
    if (wave == 0) {
      int t = 0, u = 0;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          dwF1[i][j] += red[64 * (t++)];
          dwF2[i][j] += red[64 * (t++)];
          dwG1[i][j] += red[64 * (t++)];
          if (!G2_LDS) dwG2[i][j] += red[64 * (t++)];
        }
        dbF1[i] += redb[64 * (u++)];
        dbF2[i] += redb[64 * (u++)];
        dbG1[i] += redb[64 * (u++)];
        dbG2[i] += redb[64 * (u++)];
      }
    }
    __syncthreads();
  }
  if (wave == 0) {
  // layer order in dw1 / dw2: sub-MLP F is row block 0, G is row block 1 of this coupling block
  float* gw1 = a.dw1 + (size_t)2 * kb * H * H;
  float* gw2 = a.dw2 + (size_t)2 * kb * H * H;
  float* gb1 = a.db1 ? a.db1 + (size_t)2 * kb * H : nullptr;
  float* gb2 = a.db2 ? a.db2 + (size_t)2 * kb * H : nullptr;
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      flush_tile<false, WIDE>(gw1, H, i, j, lane, dwF1[i][j]);
      flush_tile<WIDE, false>(gw2, H, i, j, lane, dwF2[i][j]);
      flush_tile<false, WIDE>(gw1 + (size_t)H * H, H, i, j, lane, dwG1[i][j]);
      if (G2_LDS) {
        constexpr int PER_WAVE = MT * MT * 64;
        const int at = (i * MT + j) * 64 + lane;  // wave 0's g2acc is the first of the four
        dwG2[i][j] = (g2acc[at] + g2acc[PER_WAVE + at]) + (g2acc[2 * PER_WAVE + at] + g2acc[3 * PER_WAVE + at]);
      }
      flush_tile<WIDE, false>(gw2 + (size_t)H * H, H, i, j, lane, dwG2[i][j]);
    }
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    flush_db_rev(gb1, H, i, lane, dbF1[i]);
    flush_db_rev(gb1 ? gb1 + H : nullptr, H, i, lane, dbG1[i]);
    flush_db_rev<WIDE>(gb2, H, i, lane, dbF2[i]);
    flush_db_rev<WIDE>(gb2 ? gb2 + H : nullptr, H, i, lane, dbG2[i]);
  }
  }
  // wave 0 has read the other waves' LDS accumulators and the reduction area: both are rewritten for the next coupling
  __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------
static int rev_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) cus = p.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

static int rev_validate(int64_t rows, int half, int blocks, int act, int dtype) {
  NF_REQUIRE(rows >= 0, NF_EINVAL, "rows negative");
  NF_REQUIRE(half >= 1 && half <= 64, NF_EINVAL, "half=%d outside 1..64", half);
  NF_REQUIRE(blocks >= 1, NF_EINVAL, "blocks=%d must be >= 1", blocks);
  NF_REQUIRE(act >= NF_ACT_NONE && act <= NF_ACT_GELU, NF_EINVAL, "unknown activation %d", act);
  NF_REQUIRE(dtype == NF_F16 || dtype == NF_BF16, NF_EUNSUPPORTED,
             "dtype code %d: the reversible MLP kernels take float16 or bfloat16 storage", dtype);
  return 0;
}

constexpr int64_t SPLIT_MIN_ROWS = 4096;  // from here on a ragged end is worth a launch of its own

static bool vec8_ok(const void* p, int64_t stride, int half) {
  return ((uintptr_t)p % 8 == 0) && (stride % 4 == 0) && (half % 4 == 0);
}
static bool vec16_ok(const void* p, int64_t stride) { return ((uintptr_t)p % 16 == 0) && (stride % 8 == 0); }

template <typename T, int HP>
static int launch_rev_fwd(RevArgs a, hipStream_t s) {
  constexpr int LAYER = (HP / 16) * (HP / 32) * RFRAG;
  const size_t lds = (size_t)a.nblocks * 4 * LAYER * 2 + (size_t)a.nblocks * 4 * HP * 4;
  const int64_t chunks = (a.rows + 31) / 32;
  // weights of several blocks leave room for one workgroup per CU only: give it 12 waves to keep three per SIMD
  const int waves = lds > 80 * 1024 ? 12 : 4;
  int64_t blocks = (chunks + waves - 1) / waves;
  const int64_t cap = (int64_t)rev_cus() * (lds > 80 * 1024 ? 1 : 2);
  if (blocks > cap) blocks = cap;
  // full-width, aligned, unragged calls of GELU, ReLU and SiLU take the variants without per-tile checks
  const bool fast = a.half == HP && a.rows % 32 == 0 && a.vec_in && a.vec_out;
  const void* kern = a.act == NF_ACT_GELU   ? (fast ? (const void*)rev_fwd_k<T, HP, NF_ACT_GELU, true>
                                                    : (const void*)rev_fwd_k<T, HP, NF_ACT_GELU, false>)
                     : a.act == NF_ACT_RELU ? (fast ? (const void*)rev_fwd_k<T, HP, NF_ACT_RELU, true>
                                                    : (const void*)rev_fwd_k<T, HP, NF_ACT_RELU, false>)
                     : (a.act == NF_ACT_SILU && fast) ? (const void*)rev_fwd_k<T, HP, NF_ACT_SILU, true>
                                            : (const void*)rev_fwd_k<T, HP, -1, false>;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  void* args[] = {(void*)&a};
  const hipError_t e = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(64 * waves), args, lds, s);
  if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(rev_fwd): %s", hipGetErrorString(e));
  return check_launch("rev_fwd");
}

template <typename T, int HP>
static int launch_rev_bwd(RevArgs a, hipStream_t s) {
  constexpr int LAYER = (HP / 16) * (HP / 32) * RFRAG;
  size_t lds = (size_t)8 * LAYER * 2 + (size_t)4 * HP * 4 + (HP > 32 ? (size_t)4 * (HP / 16) * (HP / 16) * 64 * 16 : 0);
  // the closing reduction over the waves reuses the front of LDS: the register accumulators and 4 bias sums per tile row
  const size_t red = (size_t)(HP > 32 ? 3 : 4) * (HP / 16) * (HP / 16) * 64 * 16 + (size_t)4 * (HP / 16) * 64 * 4;
  if (HP <= 32 && lds < red) lds = red;
  const int64_t chunks = (a.rows + 31) / 32;
  int64_t blocks = (chunks + 3) / 4;
  // the weight-gradient accumulators take most of the register file: one wave per SIMD
  const int64_t cap = (int64_t)rev_cus();
  if (blocks > cap) blocks = cap;
  const bool fast = a.half == HP && a.rows % 32 == 0 && a.vec_in && a.vec_out && a.vec_dy && a.vec_dx && a.wide_ok;
  const void* kern = a.act == NF_ACT_GELU   ? (fast ? (const void*)rev_bwd_block_k<T, HP, NF_ACT_GELU, true>
                                                    : (const void*)rev_bwd_block_k<T, HP, NF_ACT_GELU, false>)
                     : a.act == NF_ACT_RELU ? (fast ? (const void*)rev_bwd_block_k<T, HP, NF_ACT_RELU, true>
                                                    : (const void*)rev_bwd_block_k<T, HP, NF_ACT_RELU, false>)
                     : (a.act == NF_ACT_SILU && fast) ? (const void*)rev_bwd_block_k<T, HP, NF_ACT_SILU, true>
                                            : (const void*)rev_bwd_block_k<T, HP, -1, false>;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  void* args[] = {(void*)&a};
  const hipError_t e = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(256), args, lds, s);
  if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(rev_bwd_block): %s", hipGetErrorString(e));
  return check_launch("rev_bwd_block");
}

}  // namespace nf

using namespace nf;

extern "C" int nf_revmlp_fwd(const void* x, int64_t x_stride, void* y, int64_t y_stride, const void* w1, const void* b1,
                             const void* w2, const void* b2, int64_t rows, int half, int blocks, int act, int dtype,
                             void* stream) {
  if (int rc = rev_validate(rows, half, blocks, act, dtype)) return rc;
  if (rows == 0) return 0;
  NF_REQUIRE(x && y && w1 && w2, NF_EINVAL, "NULL pointer argument");
  NF_REQUIRE(x_stride >= 2 * half && y_stride >= 2 * half, NF_EINVAL, "row stride smaller than 2*half");
  // Rows are independent: a large batch with a ragged end runs as its multiple of 32 rows (the variants without per-tile
  // checks, where the rest of the call allows them) plus a call of its own for the last rows.
  if (rows >= SPLIT_MIN_ROWS && rows % 32 != 0) {
    const int64_t main_rows = rows - rows % 32;
    if (int rc = nf_revmlp_fwd(x, x_stride, y, y_stride, w1, b1, w2, b2, main_rows, half, blocks, act, dtype, stream)) return rc;
    return nf_revmlp_fwd((const uint16_t*)x + main_rows * x_stride, x_stride, (uint16_t*)y + main_rows * y_stride, y_stride, w1, b1, w2, b2,
                         rows - main_rows, half, blocks, act, dtype, stream);
  }
  hipStream_t s = (hipStream_t)stream;
  const int es = 2;
  for (int k0 = 0; k0 < blocks; k0 += FWD_GROUP) {
    RevArgs a = {};
    // the first group reads x; later groups continue in place on y (a wave reads its rows before it writes them)
    a.in = (const uint16_t*)(k0 == 0 ? x : y);
    a.in_stride = k0 == 0 ? x_stride : y_stride;
    a.out = (uint16_t*)y;
    a.out_stride = y_stride;
    a.w1 = (const uint16_t*)w1 + (size_t)2 * k0 * half * half;
    a.w2 = (const uint16_t*)w2 + (size_t)2 * k0 * half * half;
    a.b1 = b1 ? (const uint16_t*)b1 + (size_t)2 * k0 * half : nullptr;
    a.b2 = b2 ? (const uint16_t*)b2 + (size_t)2 * k0 * half : nullptr;
    a.rows = rows;
    a.half = half;
    a.nblocks = blocks - k0 < FWD_GROUP ? blocks - k0 : FWD_GROUP;
    a.act = act;
    a.vec_in = vec8_ok(a.in, a.in_stride, half);
    a.vec_out = vec8_ok(a.out, a.out_stride, half);
    (void)es;
    int rc;
    if (half <= 32)
      rc = dtype == NF_BF16 ? launch_rev_fwd<BF16, 32>(a, s) : launch_rev_fwd<F16, 32>(a, s);
    else
      rc = dtype == NF_BF16 ? launch_rev_fwd<BF16, 64>(a, s) : launch_rev_fwd<F16, 64>(a, s);
    if (rc) return rc;
  }
  return 0;
}

extern "C" int nf_revmlp_bwd(const void* y, int64_t y_stride, const void* dy, int64_t dy_stride, void* dx, int64_t dx_stride,
                             void* x_rec, int64_t x_rec_stride, const void* w1, const void* b1, const void* w2,
                             const void* b2, float* dw1, float* db1, float* dw2, float* db2, int64_t rows, int half,
                             int blocks, int act, int dtype, void* stream) {
  if (int rc = rev_validate(rows, half, blocks, act, dtype)) return rc;
  if (rows == 0) return 0;
  NF_REQUIRE(y && dy && dx && x_rec && w1 && w2 && dw1 && dw2, NF_EINVAL,
             "NULL pointer argument (x_rec is required: it carries the reconstructed input between blocks)");
  NF_REQUIRE(y_stride >= 2 * half && dy_stride >= 2 * half && dx_stride >= 2 * half && x_rec_stride >= 2 * half, NF_EINVAL,
             "row stride smaller than 2*half");
  // a ragged end as a call of its own (see nf_revmlp_fwd): both calls add into the same weight-gradient accumulators
  if (rows >= SPLIT_MIN_ROWS && rows % 32 != 0) {
    const int64_t m = rows - rows % 32;
    if (int rc = nf_revmlp_bwd(y, y_stride, dy, dy_stride, dx, dx_stride, x_rec, x_rec_stride, w1, b1, w2, b2, dw1, db1, dw2, db2, m, half,
                               blocks, act, dtype, stream))
      return rc;
    return nf_revmlp_bwd((const uint16_t*)y + m * y_stride, y_stride, (const uint16_t*)dy + m * dy_stride, dy_stride,
                         (uint16_t*)dx + m * dx_stride, dx_stride, (uint16_t*)x_rec + m * x_rec_stride, x_rec_stride, w1, b1, w2, b2, dw1, db1,
                         dw2, db2, rows - m, half, blocks, act, dtype, stream);
  }
  hipStream_t s = (hipStream_t)stream;
  // Full-width, aligned, unragged calls of GELU, ReLU and SiLU take one launch that walks all couplings, last
  // first (the first reads (y, dy), the others continue in place on (x_rec, dx)); anything else one launch per coupling.
  const int hp = half <= 32 ? 32 : 64;
  const bool fused = half == hp && rows % 32 == 0 && (act == NF_ACT_GELU || act == NF_ACT_RELU || act == NF_ACT_SILU) && vec8_ok(y, y_stride, half) &&
                     vec8_ok(x_rec, x_rec_stride, half) && vec8_ok(dy, dy_stride, half) && vec8_ok(dx, dx_stride, half) &&
                     vec16_ok(y, y_stride) && vec16_ok(x_rec, x_rec_stride) && vec16_ok(dy, dy_stride) && vec16_ok(dx, dx_stride);
  for (int k = blocks - 1; k >= 0; --k) {
    RevArgs a = {};
    const bool first = k == blocks - 1;
    const int kw = fused ? 0 : k;  // the fused launch offsets per coupling itself
    a.in = (const uint16_t*)(first ? y : x_rec);
    a.in_stride = first ? y_stride : x_rec_stride;
    a.out = (uint16_t*)x_rec;
    a.out_stride = x_rec_stride;
    a.dy = (const uint16_t*)(first ? dy : dx);
    a.dy_stride = first ? dy_stride : dx_stride;
    a.dx = (uint16_t*)dx;
    a.dx_stride = dx_stride;
    a.w1 = (const uint16_t*)w1 + (size_t)2 * kw * half * half;
    a.w2 = (const uint16_t*)w2 + (size_t)2 * kw * half * half;
    a.b1 = b1 ? (const uint16_t*)b1 + (size_t)2 * kw * half : nullptr;
    a.b2 = b2 ? (const uint16_t*)b2 + (size_t)2 * kw * half : nullptr;
    a.dw1 = dw1 + (size_t)2 * kw * half * half;
    a.dw2 = dw2 + (size_t)2 * kw * half * half;
    a.db1 = db1 ? db1 + (size_t)2 * kw * half : nullptr;
    a.db2 = db2 ? db2 + (size_t)2 * kw * half : nullptr;
    a.rows = rows;
    a.half = half;
    a.nblocks = fused ? blocks : 1;
    a.act = act;
    a.vec_in = vec8_ok(a.in, a.in_stride, half);
    a.vec_out = vec8_ok(a.out, a.out_stride, half);
    a.vec_dy = vec8_ok(a.dy, a.dy_stride, half);
    a.vec_dx = vec8_ok(a.dx, a.dx_stride, half);
    a.wide_ok = fused;  // the unchecked kernel is the fused launch's
    int rc;
    if (half <= 32)
      rc = dtype == NF_BF16 ? launch_rev_bwd<BF16, 32>(a, s) : launch_rev_bwd<F16, 32>(a, s);
    else
      rc = dtype == NF_BF16 ? launch_rev_bwd<BF16, 64>(a, s) : launch_rev_bwd<F16, 64>(a, s);
    if (rc || fused) return rc;
  }
  return 0;
}
