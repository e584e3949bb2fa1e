// Fused-MLP backward kernels specialised for one hidden layer (in -> H -> H -> out: the shape of neural-field
// decoders and of the benchmark, 32 -> 64 -> 64 -> 16) and, for ReLU nets of width 64, for two or three.
//
// Same algorithm as mlp_bwd_k (fused_mlp.hip) with everything static:
//   * the hidden activations stay in registers as the next layer's B fragments; for ReLU they are the gates as well;
//   * the products that contract over rows (dW = dz^T h) need both operands with the rows along K.  Two ways to get
//     them from the row-per-lane fragments: a matrix-core product with a 0/1 selector (transpose_tile: exact, one
//     MFMA per 16x16 tile, nothing through LDS), or parking the fragments in LDS and reading them back with gfx950's
//     transposing reads (tr_operand; template flag TR), which takes a third of the matrix instructions and the
//     packing of their results out of the chunk body and frees ~100 registers.  With TR the benchmark shape fits two
//     waves per SIMD (WAVES = 8, 32-row chunks): 84.8 -> 65.8 us at 2^20 rows;
//   * all weight gradients live in float32 accumulators for the wave's whole row loop; bias gradients are
//     two-element dot products of the transposed dz fragments with ones (compiled out when not asked for, DB);
//   * the waves' accumulators are summed through LDS at the end and leave as one pass of atomics per workgroup.
#pragma once

#include "fused_mlp.h"

namespace nf {

// Bias gradient of feature 16*mt + n: the four lane groups hold partial sums over disjoint rows.
__device__ __forceinline__ void flush_db(float* db, int dim, int mt, int lane, float v, bool store = false) {
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 32);
  const int f = 16 * mt + lane;
  if (db != nullptr && lane < 16 && f < dim) {
    if (store) db[f] = v;
    else unsafeAtomicAdd(db + f, v);
  }
}

typedef short s16x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));

// ReLU on a packed pair of 16-bit floats: as signed integers, negative floats (sign bit set, -0 included)
// are below zero and non-negative floats are unchanged, so one v_pk_max_i16 does both halves.
__device__ __forceinline__ uint32_t relu_pk(uint32_t p) {
  const s16x2_t z = {0, 0};
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(s16x2_t, p), z));
}
// dz = (h != 0) ? dh : 0 on packed pairs, h being a ReLU output (non-negative, never -0):
// min(h, 1) as unsigned halves is the 0/1 gate, an integer multiply applies it.  The min goes through an
// asm statement so that the optimiser does not turn the pair of packed ops back into per-half selects;
// its result only feeds the multiply, which the compiler emits (and tracks for hazards) itself.
__device__ __forceinline__ uint32_t relu_gate_pk(uint32_t dh, uint32_t h) {
  uint32_t m;
  asm("v_pk_min_u16 %0, %1, 1 op_sel_hi:[1,0]" : "=v"(m) : "v"(h));
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2_t, dh) * __builtin_bit_cast(u16x2_t, m));
}

// B fragment in chain order straight from global memory: lane (n, g) gets features
// 32*kc + 4*g .. +3 and 32*kc + 16 + 4*g .. +3 of row row0 + n; zero beyond `rows` / `width`.
__device__ __forceinline__ Frag load_rows_frag_chain(const uint16_t* base, int64_t stride, int64_t row0, int64_t rows,
                                                     int width, int kc, int lane, bool vec_ok) {
  Frag f;
  f.u = make_uint4(0u, 0u, 0u, 0u);
  const int64_t r = row0 + (lane & 15);
  if (r >= rows) return f;
  const int c0 = 32 * kc + 4 * (lane >> 4);
  const uint16_t* p = base + r * stride + c0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int c = c0 + 16 * h;
    if (vec_ok && c + 4 <= width) {
      const uint2 v = *reinterpret_cast<const uint2*>(p + 16 * h);
      f.w[2 * h] = v.x;
      f.w[2 * h + 1] = v.y;
    } else if (c < width) {
      uint16_t t[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) t[j] = (c + j < width) ? p[16 * h + j] : (uint16_t)0;
      f.w[2 * h] = (uint32_t)t[0] | ((uint32_t)t[1] << 16);
      f.w[2 * h + 1] = (uint32_t)t[2] | ((uint32_t)t[3] << 16);
    }
  }
  return f;
}

// Same fragment for the aligned case (8-byte aligned rows, width a multiple of 4): no branches, addresses of
// lanes past the end of the batch or of the row are clamped in range and their data replaced by zero.
__device__ __forceinline__ Frag load_rows_frag_chain_fast(const uint16_t* base, int64_t stride, int64_t row0, int64_t rows,
                                                          int width, int kc, int lane) {
  const int64_t r = row0 + (lane & 15);
  const int c0 = 32 * kc + 4 * (lane >> 4);
  const bool row_ok = r < rows;
  const bool lo_ok = row_ok && c0 < width, hi_ok = row_ok && c0 + 16 < width;
  const uint16_t* p = base + (row_ok ? r : 0) * stride;
  const uint2 lo = *reinterpret_cast<const uint2*>(p + (lo_ok ? c0 : 0));
  const uint2 hi = *reinterpret_cast<const uint2*>(p + (hi_ok ? c0 + 16 : 0));
  Frag f;
  f.w[0] = lo_ok ? lo.x : 0u;
  f.w[1] = lo_ok ? lo.y : 0u;
  f.w[2] = hi_ok ? hi.x : 0u;
  f.w[3] = hi_ok ? hi.y : 0u;
  return f;
}

// Store of an accumulator tile for the aligned case (width a multiple of 4, 8-byte aligned rows).
template <typename T>
__device__ __forceinline__ void store_rows_tile_fast(uint16_t* base, int64_t stride, int64_t row0, int64_t rows, int width,
                                                     int mt, int lane, f32x4_t v) {
  const int64_t r = row0 + (lane & 15);
  const int c0 = 16 * mt + 4 * (lane >> 4);
  uint2 o;
  o.x = pack2<T>(v[0], v[1]);
  o.y = pack2<T>(v[2], v[3]);
  if (r < rows && c0 < width) *reinterpret_cast<uint2*>(base + r * stride + c0) = o;
}

template <bool FAST>
__device__ __forceinline__ Frag load_chain(const uint16_t* base, int64_t stride, int64_t row0, int64_t rows, int width,
                                           int kc, int lane, bool vec_ok) {
  if (FAST) return load_rows_frag_chain_fast(base, stride, row0, rows, width, kc, lane);
  return load_rows_frag_chain(base, stride, row0, rows, width, kc, lane, vec_ok);
}

// ---- rows behind a buffer descriptor -------------------------------------------------------
// A row-major 16-bit tensor whose extent is below 2^31 bytes, addressed through a buffer resource: a lane's offset
// is 32 bits (its row and 8-byte piece, fixed for the whole launch) plus the chunk's offset, one add per load, and
// the hardware answers reads past the tensor's end with zero and drops such stores, so ragged last chunks need no
// predicates.  Pieces that lie beyond the row's width get an offset that stays past the end (OUT_OF_RANGE).
typedef unsigned int buf_v2u __attribute__((ext_vector_type(2)));
constexpr uint32_t OUT_OF_RANGE = 0x80000000u;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t rows_rsrc(const void* base, int64_t rows, int64_t stride) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)(rows * stride * 2), 0x00020000);
}
// What a launch needs of a tensor's extent for these 32-bit offsets to be safe: the tensor itself below 2^31 bytes
// (the descriptor's range check then catches every row past the end), and the furthest row any lane ever addresses
// -- the rows a partly filled last chunk pads to, and the chunks the prefetch asks for up to two grid-strides ahead (a
// stride is at most 256 workgroups x 12 waves x 32 rows) -- still below 2^32 bytes, so that no offset wraps back into range.
inline bool rows_in_reach(int64_t rows, int64_t stride) {
  const int64_t ahead = (int64_t)2 * 256 * 12 * 32 + 64;
  return rows * stride * 2 <= (((int64_t)1 << 31) - 1) && (rows + ahead) * stride * 2 + 128 < ((int64_t)1 << 32);
}
// byte offset of the piece (columns col .. col + 3) of row `row` of the first chunk
__device__ __forceinline__ uint32_t piece_offset(int row, int col, int width, int64_t stride) {
  return col < width ? (uint32_t)(((int64_t)row * stride + col) * 2) : OUT_OF_RANGE;
}

// 16-row tiles per chunk.
#ifndef NF_BWD2_NT
#define NF_BWD2_NT 4
#endif
// Workgroups per CU the ReLU kernel is compiled for.
#ifndef NF_BWD2_OCC
#define NF_BWD2_OCC 1
#endif
// dx tile in the type x is stored in
template <typename XT, bool FAST>
__device__ __forceinline__ void store_dx(const MlpArgs& a, int64_t row0, int mt, int lane, f32x4_t v) {
  if (FAST) store_rows_tile_fast<XT>(a.dx, a.dx_stride, row0, a.rows, a.d_in, mt, lane, v);
  else store_rows_tile<XT>(a.dx, a.dx_stride, row0, a.rows, a.d_in, mt, lane, v, a.dx_vec);
}

// acc[nt][mt] = bias (or 0) + W(frags) * in[nt][kc], one weight fragment read per NT products; K chunks outermost, so
// that the products into one accumulator tile are MT * NT instructions apart
// BIAS: 1 = `bias` points at the layer's staged bias row, 0 = the accumulators start at zero, -1 = decided by testing
// the pointer at run time.  The compile-time forms keep the chunk body in one basic block per layer sequence, which
// the kernels that overlap LDS round trips with matrix products need (a run-time test splits the body at every layer
// and nothing moves across); the older kernels keep the run-time test they were tuned with.
template <typename T, int NT, int MT, int KC, int BIAS = -1>
__device__ __forceinline__ void layer_nt(f32x4_t (&acc)[NT][4], const Frag (&in)[NT][2], const uint16_t* frags, const float* bias,
                                         int lane) {
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    f32x4_t b4 = {0.0f, 0.0f, 0.0f, 0.0f};
    if (BIAS == 1 || (BIAS == -1 && bias != nullptr)) b4 = *reinterpret_cast<const f32x4_t*>(bias + 16 * mt + 4 * (lane >> 4));
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt][mt] = b4;
  }
#pragma unroll
  for (int kc = 0; kc < KC; ++kc)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const Frag w = lds_frag(frags, mt * KC + kc, lane);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[nt][mt] = mfma16<T>(w, in[nt][kc], acc[nt][mt]);
    }
}

// Four parked copies of every gradient tile and bias row must fit LDS for the one-step sum of the waves.
constexpr bool bwd2_parallel_sum(int tiles, int nbias) { return 4 * (tiles * 1024 + nbias * 256) <= 160 * 1024; }

// NT: 16-row tiles per chunk (2 or 4).  Four give the scheduler two independent 32-row groups to interleave.
// XC: how x / dx are stored (MlpArgs::x_conv), fixed at compile time so that the usual case pays nothing for it;
// XC == 3: stored like the weights, and the network's activation is applied to x as it is loaded (MlpArgs::in_act).
// TR: the operands of the weight-gradient products come from LDS transposing reads (tr_operand) instead of matrix-core
// transposes.
// WAVES: waves per workgroup, 4 (one per SIMD) or 8 (two per SIMD: each then has half the register file).
// BUF: x, dy and dx are addressed through buffer descriptors (needs FAST's alignment and extents below 2^31 bytes).
// DB: bias gradients are wanted (false: the row sums are left out; the caller passed no db pointers).
template <typename T, int KIN, int HP, int OUTP, bool RELU, bool FAST, int NT, int XC, bool TR = false, int WAVES = 4, bool BUF = false, bool DB = true>
__global__ __launch_bounds__(64 * WAVES, 1) void mlp_bwd2_k(MlpArgs a) {
  constexpr int KC_IN = KIN / 32, KC_H = HP / 32, MT_H = HP / 16, MT_I = KIN / 16, MT_O = OUTP / 16;
  constexpr int KC_O = (OUTP + 31) / 32;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x;
  constexpr int nthreads = 64 * WAVES;  // the launch's workgroup size: constant trip counts let the staging loads be issued together
  const int lane = tid & 63, wave = tid >> 6;

  // the first chunk's rows are requested before the weights are staged
  constexpr int ROWS = 16 * NT;  // rows per chunk: NT / 2 independent groups of 32 rows
  const int64_t n_chunks = (a.rows + ROWS - 1) / ROWS;
  const int64_t wave_stride = (int64_t)gridDim.x * WAVES;
  const int64_t first_chunk = (int64_t)blockIdx.x * WAVES + wave;
  Frag nx[NT][KC_IN], ndy[NT][KC_O];
  // BUF: descriptors and this lane's piece offsets inside the first chunk (chain order: columns 32 kc + 16 half + 4 g)
  const __amdgpu_buffer_rsrc_t rs_x = rows_rsrc(a.x, a.rows, a.x_stride), rs_dy = rows_rsrc(a.dy, a.rows, a.dy_stride),
                               rs_dx = rows_rsrc(a.dx, a.dx != nullptr ? a.rows : 0, a.dx_stride);
  constexpr int DY_HALVES = OUTP > 16 ? 2 : 1;  // a 16-wide output has no columns 16 ..
  uint32_t off_x[KC_IN][2], off_dy[KC_O][DY_HALVES], off_dx[MT_I];
#pragma unroll
  for (int kc = 0; kc < KC_IN; ++kc)
#pragma unroll
    for (int h = 0; h < 2; ++h) off_x[kc][h] = piece_offset(lane & 15, 32 * kc + 16 * h + 4 * (lane >> 4), a.d_in, a.x_stride);
#pragma unroll
  for (int kc = 0; kc < KC_O; ++kc)
#pragma unroll
    for (int h = 0; h < DY_HALVES; ++h) off_dy[kc][h] = piece_offset(lane & 15, 32 * kc + 16 * h + 4 * (lane >> 4), a.d_out, a.dy_stride);
#pragma unroll
  for (int mt = 0; mt < MT_I; ++mt) off_dx[mt] = piece_offset(lane & 15, 16 * mt + 4 * (lane >> 4), a.d_in, a.dx_stride);
  // rows of a chunk: tile nt starts (chunk * ROWS + 16 nt) rows into the tensor (a uniform value)
  auto load_x = [&](int64_t chunk, int nt, int kc) {
    if constexpr (BUF) {
      const uint32_t at = (uint32_t)((chunk * ROWS + 16 * nt) * a.x_stride * 2);
      const buf_v2u lo = __builtin_amdgcn_raw_buffer_load_b64(rs_x, off_x[kc][0] + at, 0, 0);
      const buf_v2u hi = __builtin_amdgcn_raw_buffer_load_b64(rs_x, off_x[kc][1] + at, 0, 0);
      Frag f;
      f.w[0] = lo[0]; f.w[1] = lo[1]; f.w[2] = hi[0]; f.w[3] = hi[1];
      return f;
    } else {
      return load_chain<FAST>(a.x, a.x_stride, chunk * ROWS + 16 * nt, a.rows, a.d_in, kc, lane, a.x_vec);
    }
  };
  auto load_dy = [&](int64_t chunk, int nt, int kc) {
    if constexpr (BUF) {
      const uint32_t at = (uint32_t)((chunk * ROWS + 16 * nt) * a.dy_stride * 2);
      const buf_v2u lo = __builtin_amdgcn_raw_buffer_load_b64(rs_dy, off_dy[kc][0] + at, 0, 0);
      Frag f;
      f.w[0] = lo[0]; f.w[1] = lo[1]; f.w[2] = 0u; f.w[3] = 0u;
      if constexpr (DY_HALVES == 2) {
        const buf_v2u hi = __builtin_amdgcn_raw_buffer_load_b64(rs_dy, off_dy[kc][DY_HALVES - 1] + at, 0, 0);
        f.w[2] = hi[0]; f.w[3] = hi[1];
      }
      return f;
    } else {
      return load_chain<FAST>(a.dy, a.dy_stride, chunk * ROWS + 16 * nt, a.rows, a.d_out, kc, lane, a.dy_vec);
    }
  };
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
    for (int kc = 0; kc < KC_IN; ++kc) nx[nt][kc] = load_x(first_chunk, nt, kc);
#pragma unroll
    for (int kc = 0; kc < KC_O; ++kc) ndy[nt][kc] = load_dy(first_chunk, nt, kc);
  }

  uint16_t* f_in = reinterpret_cast<uint16_t*>(smem);          // W_in    [MT_H][KC_IN]
  uint16_t* f_hid = f_in + MT_H * KC_IN * FRAG_ELEMS;          // W_hid   [MT_H][KC_H]
  uint16_t* t_in = f_hid + MT_H * KC_H * FRAG_ELEMS;           // W_in^T  [MT_I][KC_H]
  uint16_t* t_hid = t_in + MT_I * KC_H * FRAG_ELEMS;           // W_hid^T [MT_H][KC_H]
  uint16_t* t_out = t_hid + MT_H * KC_H * FRAG_ELEMS;          // W_out^T [MT_H][KC_O]
  float* bias_in = reinterpret_cast<float*>(t_out + MT_H * KC_O * FRAG_ELEMS);
  float* bias_hid = bias_in + HP;
  // TR: two panels per wave behind the weights (activations, gradients)
  uint32_t* trA = reinterpret_cast<uint32_t*>(bias_hid + HP) + (size_t)wave * NT * TR_PANEL_DWORDS;  // NT / 2 groups x 2 panels
  uint32_t* trD = trA + TR_PANEL_DWORDS;

  stage_weight_frags<true, false, nthreads>(f_in, a.w_in, a.d_hidden, a.d_in, MT_H, KC_IN, tid, nthreads);
  stage_weight_frags<true, false, nthreads>(f_hid, a.w_hid, a.d_hidden, a.d_hidden, MT_H, KC_H, tid, nthreads);
  stage_weight_frags<true, true, nthreads>(t_in, a.w_in, a.d_hidden, a.d_in, MT_I, KC_H, tid, nthreads);
  stage_weight_frags<true, true, nthreads>(t_hid, a.w_hid, a.d_hidden, a.d_hidden, MT_H, KC_H, tid, nthreads);
  stage_weight_frags<true, true, nthreads>(t_out, a.w_out, a.d_out, a.d_hidden, MT_H, KC_O, tid, nthreads);
  stage_bias<T>(bias_in, a.b_in, a.d_hidden, HP, tid, nthreads);
  stage_bias<T>(bias_hid, a.b_hid, a.d_hidden, HP, tid, nthreads);
  __syncthreads();

  f32x4_t dw_in[MT_H][MT_I], dw_hid[MT_H][MT_H], dw_out[MT_O][MT_H];
  float db_in[MT_H], db_hid[MT_H], db_out[MT_O];  // lane (feature, g): partial row sums of feature 16*tile + n
  const f32x4_t zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int i = 0; i < MT_H; ++i) {
#pragma unroll
    for (int j = 0; j < MT_I; ++j) dw_in[i][j] = zero4;
#pragma unroll
    for (int j = 0; j < MT_H; ++j) dw_hid[i][j] = zero4;
    db_in[i] = 0.0f;
    db_hid[i] = 0.0f;
  }
#pragma unroll
  for (int i = 0; i < MT_O; ++i) {
#pragma unroll
    for (int j = 0; j < MT_H; ++j) dw_out[i][j] = zero4;
    db_out[i] = 0.0f;
  }
  const Frag sel[2] = {sel_frag<T>(0, lane), sel_frag<T>(1, lane)};


  for (int64_t chunk = first_chunk; chunk < n_chunks; chunk += wave_stride) {
    const int64_t row0 = chunk * ROWS;
    Frag in[NT][2], h1[NT][2], h2[NT][2], g1[NT][2], g2[NT][2], dz[NT][2];
    Frag xraw[(XC == 3 && !RELU) ? NT : 1][2];  // x as stored, for act'(x) at the end (ReLU reads it off act(x))
    f32x4_t acc[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int kc = 0; kc < KC_IN; ++kc) {
        if constexpr (XC == 3 && RELU) {
#pragma unroll
          for (int q = 0; q < 4; ++q) in[nt][kc].w[q] = relu_pk(nx[nt][kc].w[q]);
        } else if constexpr (XC == 3) {
          xraw[nt][kc] = nx[nt][kc];
          in[nt][kc] = act_frag<T>(nx[nt][kc], a.act);
        } else {
          in[nt][kc] = XC == 0 ? nx[nt][kc] : convert_frag(nx[nt][kc], XC);
        }
        nx[nt][kc] = load_x(chunk + wave_stride, nt, kc);
      }
#pragma unroll
      for (int kc = 0; kc < KC_O; ++kc) {
        dz[nt][kc] = ndy[nt][kc];
        ndy[nt][kc] = load_dy(chunk + wave_stride, nt, kc);
      }
    }

    // ---- forward recompute: h1 = act(W_in x + b), h2 = act(W_hid h1 + b) ----
    layer_nt<T, NT, MT_H, KC_IN, TR ? 1 : -1>(acc, in, f_in, bias_in, lane);
    if (RELU) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT_H; ++mt) {
          h1[nt][mt >> 1].w[2 * (mt & 1)] = relu_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]));
          h1[nt][mt >> 1].w[2 * (mt & 1) + 1] = relu_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]));
        }
    } else {
      with_act(a.act, [&](auto act_c) {
        constexpr int ACT = decltype(act_c)::value;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT_H; ++mt) {
            uint32_t p01, p23, q01, q23;
            act_pack<T, false>(acc[nt][mt], ACT, p01, p23);
            gate_pack<T, false>(acc[nt][mt], ACT, p01, p23, q01, q23);
            g1[nt][mt >> 1].w[2 * (mt & 1)] = q01;
            g1[nt][mt >> 1].w[2 * (mt & 1) + 1] = q23;
            h1[nt][mt >> 1].w[2 * (mt & 1)] = p01;
            h1[nt][mt >> 1].w[2 * (mt & 1) + 1] = p23;
          }
      });
    }
    layer_nt<T, NT, MT_H, KC_H, TR ? 1 : -1>(acc, h1, f_hid, bias_hid, lane);
    if (RELU) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT_H; ++mt) {
          h2[nt][mt >> 1].w[2 * (mt & 1)] = relu_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]));
          h2[nt][mt >> 1].w[2 * (mt & 1) + 1] = relu_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]));
        }
    } else {
      with_act(a.act, [&](auto act_c) {
        constexpr int ACT = decltype(act_c)::value;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT_H; ++mt) {
            uint32_t p01, p23, q01, q23;
            act_pack<T, false>(acc[nt][mt], ACT, p01, p23);
            gate_pack<T, false>(acc[nt][mt], ACT, p01, p23, q01, q23);
            g2[nt][mt >> 1].w[2 * (mt & 1)] = q01;
            g2[nt][mt >> 1].w[2 * (mt & 1) + 1] = q23;
            h2[nt][mt >> 1].w[2 * (mt & 1)] = p01;
            h2[nt][mt >> 1].w[2 * (mt & 1) + 1] = p23;
          }
      });
    }

    // Gate of a hidden layer on the packed gradient: dz = dh * act'(z), into the dz fragments.
    auto apply_gates = [&](const Frag (&h)[NT][2], const Frag (&gimg)[NT][2]) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT_H; ++mt) {
          uint32_t p01, p23;
          if (RELU) {
            p01 = relu_gate_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]), h[nt][mt >> 1].w[2 * (mt & 1)]);
            p23 = relu_gate_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]), h[nt][mt >> 1].w[2 * (mt & 1) + 1]);
          } else {
            gate_apply<T, false>(acc[nt][mt], gimg[nt][mt >> 1].w[2 * (mt & 1)], gimg[nt][mt >> 1].w[2 * (mt & 1) + 1], p01, p23);
          }
          dz[nt][mt >> 1].w[2 * (mt & 1)] = p01;
          dz[nt][mt >> 1].w[2 * (mt & 1) + 1] = p23;
        }
    };
    if constexpr (TR) {
      // Every section: park the two operands of its weight-gradient product (both 32-row groups), ask for the
      // transposed fragments, run the layer product that carries the gradient on (it does not need them, so the LDS
      // round trip hides behind its matrix instructions), then the weight-gradient products.
      constexpr int G = NT / 2;
      // ---- output layer: dW_out += dy^T h2, db_out += sum dy ; dh2 = W_out^T dy ----
      {
        Frag hb[G][MT_H], da[G][MT_O];
#pragma unroll
        for (int p = 0; p < G; ++p) {
#pragma unroll
          for (int kc = 0; kc < KC_H; ++kc) {
            park_frag_rows(trA + p * 2 * TR_PANEL_DWORDS, h2[2 * p][kc], 0, kc, lane);
            park_frag_rows(trA + p * 2 * TR_PANEL_DWORDS, h2[2 * p + 1][kc], 1, kc, lane);
          }
#pragma unroll
          for (int kc = 0; kc < KC_O; ++kc) {
            park_frag_rows<(OUTP > 16)>(trD + p * 2 * TR_PANEL_DWORDS, dz[2 * p][kc], 0, kc, lane);
            park_frag_rows<(OUTP > 16)>(trD + p * 2 * TR_PANEL_DWORDS, dz[2 * p + 1][kc], 1, kc, lane);
          }
        }
#pragma unroll
        for (int p = 0; p < G; ++p) {
#pragma unroll
          for (int j = 0; j < MT_H; ++j) hb[p][j] = tr_operand(trA + p * 2 * TR_PANEL_DWORDS, j, lane);
#pragma unroll
          for (int i = 0; i < MT_O; ++i) da[p][i] = tr_operand(trD + p * 2 * TR_PANEL_DWORDS, i, lane);
        }
        layer_nt<T, NT, MT_H, KC_O, 0>(acc, dz, t_out, nullptr, lane);
#pragma unroll
        for (int p = 0; p < G; ++p)
#pragma unroll
          for (int i = 0; i < MT_O; ++i) {
#pragma unroll
            for (int j = 0; j < MT_H; ++j) dw_out[i][j] = mfma16<T>(da[p][i], hb[p][j], dw_out[i][j]);
            if constexpr (DB) {
#pragma unroll
              for (int q = 0; q < 4; ++q) db_out[i] = dot2_ones<T>(da[p][i].w[q], db_out[i]);
            }
          }
      }
      // ---- hidden layer: dz2 = dh2 * act'(z2) ; dW_hid += dz2^T h1 ; dh1 = W_hid^T dz2 ----
      apply_gates(h2, g2);
      {
        Frag hb[G][MT_H], da[G][MT_H];
#pragma unroll
        for (int p = 0; p < G; ++p)
#pragma unroll
          for (int kc = 0; kc < KC_H; ++kc) {
            park_frag_rows(trA + p * 2 * TR_PANEL_DWORDS, h1[2 * p][kc], 0, kc, lane);
            park_frag_rows(trA + p * 2 * TR_PANEL_DWORDS, h1[2 * p + 1][kc], 1, kc, lane);
            park_frag_rows(trD + p * 2 * TR_PANEL_DWORDS, dz[2 * p][kc], 0, kc, lane);
            park_frag_rows(trD + p * 2 * TR_PANEL_DWORDS, dz[2 * p + 1][kc], 1, kc, lane);
          }
#pragma unroll
        for (int p = 0; p < G; ++p)
#pragma unroll
          for (int j = 0; j < MT_H; ++j) {
            hb[p][j] = tr_operand(trA + p * 2 * TR_PANEL_DWORDS, j, lane);
            da[p][j] = tr_operand(trD + p * 2 * TR_PANEL_DWORDS, j, lane);
          }
        layer_nt<T, NT, MT_H, KC_H, 0>(acc, dz, t_hid, nullptr, lane);
#pragma unroll
        for (int p = 0; p < G; ++p)
#pragma unroll
          for (int i = 0; i < MT_H; ++i) {
#pragma unroll
            for (int j = 0; j < MT_H; ++j) dw_hid[i][j] = mfma16<T>(da[p][i], hb[p][j], dw_hid[i][j]);
            if constexpr (DB) {
#pragma unroll
              for (int q = 0; q < 4; ++q) db_hid[i] = dot2_ones<T>(da[p][i].w[q], db_hid[i]);
            }
          }
      }
      // ---- input layer: dz1 = dh1 * act'(z1) ; dW_in += dz1^T x ; dx = W_in^T dz1 ----
      apply_gates(h1, g1);
      {
        Frag xb[G][MT_I], da[G][MT_H];
#pragma unroll
        for (int p = 0; p < G; ++p) {
#pragma unroll
          for (int kc = 0; kc < KC_IN; ++kc) {
            park_frag_rows(trA + p * 2 * TR_PANEL_DWORDS, in[2 * p][kc], 0, kc, lane);
            park_frag_rows(trA + p * 2 * TR_PANEL_DWORDS, in[2 * p + 1][kc], 1, kc, lane);
          }
#pragma unroll
          for (int kc = 0; kc < KC_H; ++kc) {
            park_frag_rows(trD + p * 2 * TR_PANEL_DWORDS, dz[2 * p][kc], 0, kc, lane);
            park_frag_rows(trD + p * 2 * TR_PANEL_DWORDS, dz[2 * p + 1][kc], 1, kc, lane);
          }
        }
#pragma unroll
        for (int p = 0; p < G; ++p) {
#pragma unroll
          for (int j = 0; j < MT_I; ++j) xb[p][j] = tr_operand(trA + p * 2 * TR_PANEL_DWORDS, j, lane);
#pragma unroll
          for (int i = 0; i < MT_H; ++i) da[p][i] = tr_operand(trD + p * 2 * TR_PANEL_DWORDS, i, lane);
        }
        if (a.dx != nullptr) layer_nt<T, NT, MT_I, KC_H, 0>(acc, dz, t_in, nullptr, lane);
#pragma unroll
        for (int p = 0; p < G; ++p)
#pragma unroll
          for (int i = 0; i < MT_H; ++i) {
#pragma unroll
            for (int j = 0; j < MT_I; ++j) dw_in[i][j] = mfma16<T>(da[p][i], xb[p][j], dw_in[i][j]);
            if constexpr (DB) {
#pragma unroll
              for (int q = 0; q < 4; ++q) db_in[i] = dot2_ones<T>(da[p][i].w[q], db_in[i]);
            }
          }
      }
    } else {
    // ---- output layer: dW_out += dy^T h2, db_out += sum dy ; dh2 = W_out^T dy ----
#pragma unroll
    for (int p = 0; p < NT / 2; ++p) {
      Frag hb[MT_H];
#pragma unroll
      for (int j = 0; j < MT_H; ++j)
        hb[j] = transpose_tile<T>(h2[2 * p][j >> 1], h2[2 * p + 1][j >> 1], sel[j & 1]);
#pragma unroll
      for (int i = 0; i < MT_O; ++i) {
        const Frag da = transpose_tile<T>(dz[2 * p][i >> 1], dz[2 * p + 1][i >> 1], sel[i & 1]);
#pragma unroll
        for (int j = 0; j < MT_H; ++j) dw_out[i][j] = mfma16<T>(da, hb[j], dw_out[i][j]);
#pragma unroll
        for (int q = 0; q < 4; ++q) db_out[i] = dot2_ones<T>(da.w[q], db_out[i]);
      }
    }
    layer_nt<T, NT, MT_H, KC_O>(acc, dz, t_out, nullptr, lane);
    // ---- hidden layer: dz2 = dh2 * act'(z2) ; dW_hid += dz2^T h1 ; dh1 = W_hid^T dz2 ----
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT_H; ++mt) {
        uint32_t p01, p23;
        if (RELU) {
          p01 = relu_gate_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]), h2[nt][mt >> 1].w[2 * (mt & 1)]);
          p23 = relu_gate_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]), h2[nt][mt >> 1].w[2 * (mt & 1) + 1]);
        } else {
          gate_apply<T, false>(acc[nt][mt], g2[nt][mt >> 1].w[2 * (mt & 1)], g2[nt][mt >> 1].w[2 * (mt & 1) + 1], p01, p23);
        }
        dz[nt][mt >> 1].w[2 * (mt & 1)] = p01;
        dz[nt][mt >> 1].w[2 * (mt & 1) + 1] = p23;
      }
#pragma unroll
    for (int p = 0; p < NT / 2; ++p) {
      Frag hb[MT_H];
#pragma unroll
      for (int j = 0; j < MT_H; ++j)
        hb[j] = transpose_tile<T>(h1[2 * p][j >> 1], h1[2 * p + 1][j >> 1], sel[j & 1]);
#pragma unroll
      for (int i = 0; i < MT_H; ++i) {
        const Frag da = transpose_tile<T>(dz[2 * p][i >> 1], dz[2 * p + 1][i >> 1], sel[i & 1]);
#pragma unroll
        for (int j = 0; j < MT_H; ++j) dw_hid[i][j] = mfma16<T>(da, hb[j], dw_hid[i][j]);
#pragma unroll
        for (int q = 0; q < 4; ++q) db_hid[i] = dot2_ones<T>(da.w[q], db_hid[i]);
      }
    }
    layer_nt<T, NT, MT_H, KC_H>(acc, dz, t_hid, nullptr, lane);
    // ---- input layer: dz1 = dh1 * act'(z1) ; dW_in += dz1^T x ; dx = W_in^T dz1 ----
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT_H; ++mt) {
        uint32_t p01, p23;
        if (RELU) {
          p01 = relu_gate_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]), h1[nt][mt >> 1].w[2 * (mt & 1)]);
          p23 = relu_gate_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]), h1[nt][mt >> 1].w[2 * (mt & 1) + 1]);
        } else {
          gate_apply<T, false>(acc[nt][mt], g1[nt][mt >> 1].w[2 * (mt & 1)], g1[nt][mt >> 1].w[2 * (mt & 1) + 1], p01, p23);
        }
        dz[nt][mt >> 1].w[2 * (mt & 1)] = p01;
        dz[nt][mt >> 1].w[2 * (mt & 1) + 1] = p23;
      }
#pragma unroll
    for (int p = 0; p < NT / 2; ++p) {
      Frag xb[MT_I];
#pragma unroll
      for (int j = 0; j < MT_I; ++j)
        xb[j] = transpose_tile<T>(in[2 * p][j >> 1], in[2 * p + 1][j >> 1], sel[j & 1]);
#pragma unroll
      for (int i = 0; i < MT_H; ++i) {
        const Frag da = transpose_tile<T>(dz[2 * p][i >> 1], dz[2 * p + 1][i >> 1], sel[i & 1]);
#pragma unroll
        for (int j = 0; j < MT_I; ++j) dw_in[i][j] = mfma16<T>(da, xb[j], dw_in[i][j]);
#pragma unroll
        for (int q = 0; q < 4; ++q) db_in[i] = dot2_ones<T>(da.w[q], db_in[i]);
      }
    }
      if (a.dx != nullptr) layer_nt<T, NT, MT_I, KC_H>(acc, dz, t_in, nullptr, lane);
    }
    if (a.dx != nullptr) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT_I; ++mt) {
          // chain-order fragments hold x exactly where the packed dx tiles sit
          if constexpr (XC == 3 && RELU)
            acc[nt][mt] = input_gate<T>(acc[nt][mt], in[nt][mt >> 1].w[2 * (mt & 1)], in[nt][mt >> 1].w[2 * (mt & 1) + 1], NF_ACT_RELU);
          else if constexpr (XC == 3)
            acc[nt][mt] = input_gate<T>(acc[nt][mt], xraw[nt][mt >> 1].w[2 * (mt & 1)], xraw[nt][mt >> 1].w[2 * (mt & 1) + 1], a.act);
          if constexpr (BUF) {
            buf_v2u o;
            if (XC == 1) { o[0] = pack2<F16>(acc[nt][mt][0], acc[nt][mt][1]); o[1] = pack2<F16>(acc[nt][mt][2], acc[nt][mt][3]); }
            else if (XC == 2) { o[0] = pack2<BF16>(acc[nt][mt][0], acc[nt][mt][1]); o[1] = pack2<BF16>(acc[nt][mt][2], acc[nt][mt][3]); }
            else { o[0] = pack2<T>(acc[nt][mt][0], acc[nt][mt][1]); o[1] = pack2<T>(acc[nt][mt][2], acc[nt][mt][3]); }
            __builtin_amdgcn_raw_buffer_store_b64(o, rs_dx, off_dx[mt] + (uint32_t)((row0 + 16 * nt) * a.dx_stride * 2), 0, 0);
          } else if (XC == 1) store_dx<F16, FAST>(a, row0 + 16 * nt, mt, lane, acc[nt][mt]);
          else if (XC == 2) store_dx<BF16, FAST>(a, row0 + 16 * nt, mt, lane, acc[nt][mt]);
          else store_dx<T, FAST>(a, row0 + 16 * nt, mt, lane, acc[nt][mt]);
        }
    }
  }

  constexpr int TILES = MT_H * (MT_I + MT_H) + MT_O * MT_H, NBIAS = 2 * MT_H + MT_O;
  constexpr bool PARALLEL_SUM = bwd2_parallel_sum(TILES, NBIAS);
  static_assert(WAVES == 4 || PARALLEL_SUM, "eight waves close through the parallel sum");
  if constexpr (PARALLEL_SUM) {
    // ---- sum the gradients of the waves through LDS (the weight fragments are dead by now): four waves park their
    // accumulators, then wave w adds up and flushes every fourth tile, so the atomics leave from four waves.  With
    // eight waves the upper four first hand theirs to the lower four. ----
    __syncthreads();
    f32x4_t* red = reinterpret_cast<f32x4_t*>(smem);                               // [4][TILES][64]
    float* redb = reinterpret_cast<float*>(smem) + (size_t)4 * TILES * 256;          // [4][NBIAS][64]
    // ADD = false: store this wave's accumulators into slot w; ADD = true: add slot w to them
    auto exchange = [&](int w, auto add_c) {
      constexpr bool ADD = decltype(add_c)::value;
      f32x4_t* mine = red + (size_t)w * TILES * 64 + lane;
      float* mineb = redb + (size_t)w * NBIAS * 64 + lane;
      int t = 0, u = 0;
      auto tile = [&](f32x4_t& v) {
        if (ADD) v += mine[64 * t];
        else mine[64 * t] = v;
        ++t;
      };
      auto row = [&](float& v) {
        if (ADD) v += mineb[64 * u];
        else mineb[64 * u] = v;
        ++u;
      };
#pragma unroll
      for (int i = 0; i < MT_H; ++i) {
#pragma unroll
        for (int j = 0; j < MT_I; ++j) tile(dw_in[i][j]);
#pragma unroll
        for (int j = 0; j < MT_H; ++j) tile(dw_hid[i][j]);
        row(db_in[i]);
        row(db_hid[i]);
      }
#pragma unroll
      for (int i = 0; i < MT_O; ++i) {
#pragma unroll
        for (int j = 0; j < MT_H; ++j) tile(dw_out[i][j]);
        row(db_out[i]);
      }
    };
    if constexpr (WAVES == 8) {
      if (wave >= 4) exchange(wave - 4, std::false_type{});
      __syncthreads();
      if (wave < 4) exchange(wave, std::true_type{});
      __syncthreads();
    }
    if (wave < 4) exchange(wave, std::false_type{});
    __syncthreads();
    auto tile_sum = [&](int t) {
      const f32x4_t* p = red + (size_t)t * 64 + lane;
      return (p[0] + p[(size_t)TILES * 64]) + (p[(size_t)2 * TILES * 64] + p[(size_t)3 * TILES * 64]);
    };
    auto bias_sum = [&](int u) {
      const float* p = redb + (size_t)u * 64 + lane;
      return (p[0] + p[(size_t)NBIAS * 64]) + (p[(size_t)2 * NBIAS * 64] + p[(size_t)3 * NBIAS * 64]);
    };
    {
      // where the sums go: the caller's accumulators (atomic adds), or this workgroup's own slot (plain stores)
      const bool own = a.partials != nullptr;
      float* slot = own ? a.partials + (size_t)blockIdx.x * a.partial_stride : nullptr;
      float* p_dw_in = own ? slot : a.dw_in;
      float* p_dw_hid = own ? p_dw_in + a.d_hidden * a.d_in : a.dw_hid;
      float* p_dw_out = own ? p_dw_hid + a.d_hidden * a.d_hidden : a.dw_out;
      float* p_db_in = own ? p_dw_out + a.d_out * a.d_hidden : a.db_in;
      float* p_db_hid = own ? p_db_in + a.d_hidden : a.db_hid;
      float* p_db_out = own ? p_db_hid + a.d_hidden : a.db_out;
      int t = 0, u = 0;
  #pragma unroll
      for (int i = 0; i < MT_H; ++i) {
  #pragma unroll
        for (int j = 0; j < MT_I; ++j, ++t)
          if ((t & 3) == wave) flush_dw_tile(p_dw_in, a.d_hidden, a.d_in, i, j, lane, tile_sum(t), own);
  #pragma unroll
        for (int j = 0; j < MT_H; ++j, ++t)
          if ((t & 3) == wave) flush_dw_tile(p_dw_hid, a.d_hidden, a.d_hidden, i, j, lane, tile_sum(t), own);
        if ((u & 3) == wave) flush_db(p_db_in, a.d_hidden, i, lane, bias_sum(u), own);
        ++u;
        if ((u & 3) == wave) flush_db(p_db_hid, a.d_hidden, i, lane, bias_sum(u), own);
        ++u;
      }
  #pragma unroll
      for (int i = 0; i < MT_O; ++i) {
  #pragma unroll
        for (int j = 0; j < MT_H; ++j, ++t)
          if ((t & 3) == wave) flush_dw_tile(p_dw_out, a.d_out, a.d_hidden, i, j, lane, tile_sum(t), own);
        if ((u & 3) == wave) flush_db(p_db_out, a.d_out, i, lane, bias_sum(u), own);
        ++u;
      }
    }
    return;
  }
  // ---- reduce the gradients over the four waves through LDS (the weight fragments are dead by now), then
  // one pass of atomics per workgroup ----
  __syncthreads();
  f32x4_t* red = reinterpret_cast<f32x4_t*>(smem) + lane;
  float* redb = reinterpret_cast<float*>(smem) + (size_t)(MT_H * (MT_I + MT_H) + MT_O * MT_H) * 256 + lane;
  for (int w = 1; w < 4; ++w) {
    if (wave == w) {
      int t = 0, u = 0;
#pragma unroll
      for (int i = 0; i < MT_H; ++i) {
#pragma unroll
        for (int j = 0; j < MT_I; ++j) red[64 * (t++)] = dw_in[i][j];
#pragma unroll
        for (int j = 0; j < MT_H; ++j) red[64 * (t++)] = dw_hid[i][j];
        redb[64 * (u++)] = db_in[i];
        redb[64 * (u++)] = db_hid[i];
      }
#pragma unroll
      for (int i = 0; i < MT_O; ++i) {
#pragma unroll
        for (int j = 0; j < MT_H; ++j) red[64 * (t++)] = dw_out[i][j];
        redb[64 * (u++)] = db_out[i];
      }
    }
    __syncthreads();
    if (wave == 0) {
      int t = 0, u = 0;
#pragma unroll
      for (int i = 0; i < MT_H; ++i) {
#pragma unroll
        for (int j = 0; j < MT_I; ++j) dw_in[i][j] += red[64 * (t++)];
#pragma unroll
        for (int j = 0; j < MT_H; ++j) dw_hid[i][j] += red[64 * (t++)];
        db_in[i] += redb[64 * (u++)];
        db_hid[i] += redb[64 * (u++)];
      }
#pragma unroll
      for (int i = 0; i < MT_O; ++i) {
#pragma unroll
        for (int j = 0; j < MT_H; ++j) dw_out[i][j] += red[64 * (t++)];
        db_out[i] += redb[64 * (u++)];
      }
    }
    __syncthreads();
  }
  if (wave != 0) return;
#pragma unroll
  for (int i = 0; i < MT_H; ++i) {
#pragma unroll
    for (int j = 0; j < MT_I; ++j) flush_dw_tile(a.dw_in, a.d_hidden, a.d_in, i, j, lane, dw_in[i][j]);
#pragma unroll
    for (int j = 0; j < MT_H; ++j) flush_dw_tile(a.dw_hid, a.d_hidden, a.d_hidden, i, j, lane, dw_hid[i][j]);
    flush_db(a.db_in, a.d_hidden, i, lane, db_in[i]);
    flush_db(a.db_hid, a.d_hidden, i, lane, db_hid[i]);
  }
#pragma unroll
  for (int i = 0; i < MT_O; ++i) {
#pragma unroll
    for (int j = 0; j < MT_H; ++j) flush_dw_tile(a.dw_out, a.d_out, a.d_hidden, i, j, lane, dw_out[i][j]);
    flush_db(a.db_out, a.d_out, i, lane, db_out[i]);
  }
}

// ---------------------------------------------------------------------------------------
// The same kernel for deeper ReLU nets: NH hidden-to-hidden layers (depth = NH + 1), 32-row chunks.  Every
// hidden activation of the chunk stays in registers (they are the gates as well), every weight gradient in float32
// accumulators over the wave's row loop; the weights of all layers, in both forms, are resident in LDS.
// ---------------------------------------------------------------------------------------
// hidden-to-hidden weight gradients that accumulate in LDS instead of registers
// (measured on the compiler: with two in registers the two-layer kernels spill where the input or output layer is 64
// wide, the three-layer kernels, whose third accumulator is in LDS anyway, do not)
constexpr int bwdn_lds_layers(int kin, int outp, int nh) {
  if (nh >= 3) return nh - 2;
  return (kin == 32 && outp == 16) ? 0 : 1;
}

// IA: ReLU is applied to x as it is loaded (MlpArgs::in_act) and dx is the gradient in front of that ReLU.
template <typename T, int KIN, int HP, int OUTP, int NH, bool FAST, bool IA>
__global__ __launch_bounds__(256) void mlp_bwdn_k(MlpArgs a) {
  constexpr int KC_IN = KIN / 32, KC_H = HP / 32, MT_H = HP / 16, MT_I = KIN / 16, MT_O = OUTP / 16;
  constexpr int KC_O = (OUTP + 31) / 32;
  constexpr int NT = 2;
  constexpr int HID = MT_H * KC_H * FRAG_ELEMS;  // one hidden layer's fragments
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int lane = tid & 63, wave = tid >> 6;

  uint16_t* f_in = reinterpret_cast<uint16_t*>(smem);          // W_in      [MT_H][KC_IN]
  uint16_t* f_hid = f_in + MT_H * KC_IN * FRAG_ELEMS;          // W_hid[k]  [NH][MT_H][KC_H]
  uint16_t* t_in = f_hid + NH * HID;                           // W_in^T    [MT_I][KC_H]
  uint16_t* t_hid = t_in + MT_I * KC_H * FRAG_ELEMS;           // W_hid[k]^T
  uint16_t* t_out = t_hid + NH * HID;                          // W_out^T   [MT_H][KC_O]
  float* bias_in = reinterpret_cast<float*>(t_out + MT_H * KC_O * FRAG_ELEMS);
  float* bias_hid = bias_in + HP;                              // [NH][HP]
  // One or two 64x64 hidden accumulators stay in registers next to the rest; the others live in LDS, 16 KiB per
  // wave and layer (the layers of highest index).
  constexpr int LA = bwdn_lds_layers(KIN, OUTP, NH), NREG = NH - LA;
  constexpr size_t W_BYTES = ((size_t)MT_H * KC_IN + (size_t)MT_I * KC_H + 2 * (size_t)NH * MT_H * KC_H + (size_t)MT_H * KC_O) * 1024 +
                             (size_t)(1 + NH) * HP * 4;
  constexpr size_t RED_BYTES = (size_t)(MT_H * (MT_I + NREG * MT_H) + MT_O * MT_H) * 1024 + (size_t)((1 + NH) * MT_H + MT_O) * 256;
  constexpr size_t LACC_AT = W_BYTES > RED_BYTES ? W_BYTES : RED_BYTES;  // behind the weights and the closing reduction's area
  f32x4_t* lacc = reinterpret_cast<f32x4_t*>(smem + LACC_AT) + (size_t)wave * (LA * MT_H * MT_H * 64);
  for (int i = lane; i < LA * MT_H * MT_H * 64; i += 64) lacc[i] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

  const size_t hh = (size_t)a.d_hidden * a.d_hidden;
  stage_weight_frags<true, false>(f_in, a.w_in, a.d_hidden, a.d_in, MT_H, KC_IN, tid, nthreads);
  stage_weight_frags<true, true>(t_in, a.w_in, a.d_hidden, a.d_in, MT_I, KC_H, tid, nthreads);
  stage_weight_frags<true, true>(t_out, a.w_out, a.d_out, a.d_hidden, MT_H, KC_O, tid, nthreads);
  stage_bias<T>(bias_in, a.b_in, a.d_hidden, HP, tid, nthreads);
  for (int k = 0; k < NH; ++k) {
    stage_weight_frags<true, false>(f_hid + k * HID, a.w_hid + k * hh, a.d_hidden, a.d_hidden, MT_H, KC_H, tid, nthreads);
    stage_weight_frags<true, true>(t_hid + k * HID, a.w_hid + k * hh, a.d_hidden, a.d_hidden, MT_H, KC_H, tid, nthreads);
    stage_bias<T>(bias_hid + k * HP, a.b_hid ? a.b_hid + (size_t)k * a.d_hidden : nullptr, a.d_hidden, HP, tid, nthreads);
  }
  __syncthreads();

  f32x4_t dw_in[MT_H][MT_I], dw_hid[NREG][MT_H][MT_H], dw_out[MT_O][MT_H];
  float db_in[MT_H], db_hid[NH][MT_H], db_out[MT_O];
  const f32x4_t zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int i = 0; i < MT_H; ++i) {
#pragma unroll
    for (int j = 0; j < MT_I; ++j) dw_in[i][j] = zero4;
    db_in[i] = 0.0f;
#pragma unroll
    for (int k = 0; k < NH; ++k) {
      if (k < NREG) {
#pragma unroll
        for (int j = 0; j < MT_H; ++j) dw_hid[k < NREG ? k : 0][i][j] = zero4;
      }
      db_hid[k][i] = 0.0f;
    }
  }
#pragma unroll
  for (int i = 0; i < MT_O; ++i) {
#pragma unroll
    for (int j = 0; j < MT_H; ++j) dw_out[i][j] = zero4;
    db_out[i] = 0.0f;
  }
  const Frag sel[2] = {sel_frag<T>(0, lane), sel_frag<T>(1, lane)};

  constexpr int ROWS = 16 * NT;
  const int64_t n_chunks = (a.rows + ROWS - 1) / ROWS;
  const int64_t wave_stride = (int64_t)gridDim.x * 4;
  const int64_t first_chunk = (int64_t)blockIdx.x * 4 + wave;
  Frag nx[NT][KC_IN], ndy[NT][KC_O];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
    for (int kc = 0; kc < KC_IN; ++kc)
      nx[nt][kc] = load_chain<FAST>(a.x, a.x_stride, first_chunk * ROWS + 16 * nt, a.rows, a.d_in, kc, lane, a.x_vec);
#pragma unroll
    for (int kc = 0; kc < KC_O; ++kc)
      ndy[nt][kc] = load_chain<FAST>(a.dy, a.dy_stride, first_chunk * ROWS + 16 * nt, a.rows, a.d_out, kc, lane, a.dy_vec);
  }

  for (int64_t chunk = first_chunk; chunk < n_chunks; chunk += wave_stride) {
    const int64_t row0 = chunk * ROWS;
    Frag in[NT][2], h[NH + 1][NT][2], dz[NT][2];
    f32x4_t acc[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int kc = 0; kc < KC_IN; ++kc) {
        in[nt][kc] = nx[nt][kc];
        if (IA) {
#pragma unroll
          for (int q = 0; q < 4; ++q) in[nt][kc].w[q] = relu_pk(in[nt][kc].w[q]);
        }
        nx[nt][kc] = load_chain<FAST>(a.x, a.x_stride, (chunk + wave_stride) * ROWS + 16 * nt, a.rows, a.d_in, kc, lane, a.x_vec);
      }
#pragma unroll
      for (int kc = 0; kc < KC_O; ++kc) {
        dz[nt][kc] = ndy[nt][kc];
        ndy[nt][kc] = load_chain<FAST>(a.dy, a.dy_stride, (chunk + wave_stride) * ROWS + 16 * nt, a.rows, a.d_out, kc, lane, a.dy_vec);
      }
    }
    // ---- forward recompute: h[0] = relu(W_in x + b), h[k] = relu(W_hid[k-1] h[k-1] + b) ----
    layer_nt<T, NT, MT_H, KC_IN>(acc, in, f_in, bias_in, lane);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT_H; ++mt) {
        h[0][nt][mt >> 1].w[2 * (mt & 1)] = relu_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]));
        h[0][nt][mt >> 1].w[2 * (mt & 1) + 1] = relu_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]));
      }
#pragma unroll
    for (int k = 1; k <= NH; ++k) {
      layer_nt<T, NT, MT_H, KC_H>(acc, h[k - 1], f_hid + (k - 1) * HID, bias_hid + (k - 1) * HP, lane);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT_H; ++mt) {
          h[k][nt][mt >> 1].w[2 * (mt & 1)] = relu_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]));
          h[k][nt][mt >> 1].w[2 * (mt & 1) + 1] = relu_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]));
        }
    }
    // ---- output layer: dW_out += dy^T h[NH], db_out += sum dy ; dh = W_out^T dy ----
    {
      Frag hb[MT_H];
#pragma unroll
      for (int j = 0; j < MT_H; ++j) hb[j] = transpose_tile<T>(h[NH][0][j >> 1], h[NH][1][j >> 1], sel[j & 1]);
#pragma unroll
      for (int i = 0; i < MT_O; ++i) {
        const Frag da = transpose_tile<T>(dz[0][i >> 1], dz[1][i >> 1], sel[i & 1]);
#pragma unroll
        for (int j = 0; j < MT_H; ++j) dw_out[i][j] = mfma16<T>(da, hb[j], dw_out[i][j]);
#pragma unroll
        for (int q = 0; q < 4; ++q) db_out[i] = dot2_ones<T>(da.w[q], db_out[i]);
      }
    }
    layer_nt<T, NT, MT_H, KC_O>(acc, dz, t_out, nullptr, lane);
    // ---- hidden layers, last first: dz_k = dh_k gated by h[k] ; dW_hid[k-1] += dz_k^T h[k-1] ; dh_{k-1} = W_hid[k-1]^T dz_k
#pragma unroll
    for (int k = NH; k >= 1; --k) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT_H; ++mt) {
          dz[nt][mt >> 1].w[2 * (mt & 1)] = relu_gate_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]), h[k][nt][mt >> 1].w[2 * (mt & 1)]);
          dz[nt][mt >> 1].w[2 * (mt & 1) + 1] =
              relu_gate_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]), h[k][nt][mt >> 1].w[2 * (mt & 1) + 1]);
        }
      {
        Frag hb[MT_H];
#pragma unroll
        for (int j = 0; j < MT_H; ++j) hb[j] = transpose_tile<T>(h[k - 1][0][j >> 1], h[k - 1][1][j >> 1], sel[j & 1]);
#pragma unroll
        for (int i = 0; i < MT_H; ++i) {
          const Frag da = transpose_tile<T>(dz[0][i >> 1], dz[1][i >> 1], sel[i & 1]);
          if (k - 1 < NREG) {
#pragma unroll
            for (int j = 0; j < MT_H; ++j)
              dw_hid[k - 1 < NREG ? k - 1 : 0][i][j] = mfma16<T>(da, hb[j], dw_hid[k - 1 < NREG ? k - 1 : 0][i][j]);
          } else {
#pragma unroll
            for (int j = 0; j < MT_H; ++j) {
              f32x4_t* slot = lacc + (((k - 1 - NREG) * MT_H + i) * MT_H + j) * 64 + lane;
              *slot = mfma16<T>(da, hb[j], *slot);
            }
          }
#pragma unroll
          for (int q = 0; q < 4; ++q) db_hid[k - 1][i] = dot2_ones<T>(da.w[q], db_hid[k - 1][i]);
        }
      }
      layer_nt<T, NT, MT_H, KC_H>(acc, dz, t_hid + (k - 1) * HID, nullptr, lane);
    }
    // ---- input layer: dz_0 = dh_0 gated by h[0] ; dW_in += dz_0^T x ; dx = W_in^T dz_0 ----
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT_H; ++mt) {
        dz[nt][mt >> 1].w[2 * (mt & 1)] = relu_gate_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]), h[0][nt][mt >> 1].w[2 * (mt & 1)]);
        dz[nt][mt >> 1].w[2 * (mt & 1) + 1] =
            relu_gate_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]), h[0][nt][mt >> 1].w[2 * (mt & 1) + 1]);
      }
    {
      Frag xb[MT_I];
#pragma unroll
      for (int j = 0; j < MT_I; ++j) xb[j] = transpose_tile<T>(in[0][j >> 1], in[1][j >> 1], sel[j & 1]);
#pragma unroll
      for (int i = 0; i < MT_H; ++i) {
        const Frag da = transpose_tile<T>(dz[0][i >> 1], dz[1][i >> 1], sel[i & 1]);
#pragma unroll
        for (int j = 0; j < MT_I; ++j) dw_in[i][j] = mfma16<T>(da, xb[j], dw_in[i][j]);
#pragma unroll
        for (int q = 0; q < 4; ++q) db_in[i] = dot2_ones<T>(da.w[q], db_in[i]);
      }
    }
    if (a.dx != nullptr) {
      layer_nt<T, NT, MT_I, KC_H>(acc, dz, t_in, nullptr, lane);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT_I; ++mt) {
          if (IA)  // x > 0 where relu(x), held in chain order exactly where the packed dx tile sits, is not zero
            acc[nt][mt] = input_gate<T>(acc[nt][mt], in[nt][mt >> 1].w[2 * (mt & 1)], in[nt][mt >> 1].w[2 * (mt & 1) + 1], NF_ACT_RELU);
          store_dx<T, FAST>(a, row0 + 16 * nt, mt, lane, acc[nt][mt]);
        }
    }
  }

  // ---- reduce the gradients over the four waves through LDS (the weight fragments are dead by now), then
  // one pass of atomics per workgroup ----
  __syncthreads();
  constexpr int N_TILES = MT_H * (MT_I + NREG * MT_H) + MT_O * MT_H;
  f32x4_t* red = reinterpret_cast<f32x4_t*>(smem) + lane;
  float* redb = reinterpret_cast<float*>(smem) + (size_t)N_TILES * 256 + lane;
  for (int w = 1; w < 4; ++w) {
    if (wave == w) {
      int t = 0, u = 0;
#pragma unroll
      for (int i = 0; i < MT_H; ++i) {
#pragma unroll
        for (int j = 0; j < MT_I; ++j) red[64 * (t++)] = dw_in[i][j];
        redb[64 * (u++)] = db_in[i];
#pragma unroll
        for (int k = 0; k < NH; ++k) {
          if (k < NREG) {
#pragma unroll
            for (int j = 0; j < MT_H; ++j) red[64 * (t++)] = dw_hid[k < NREG ? k : 0][i][j];
          }
          redb[64 * (u++)] = db_hid[k][i];
        }
      }
#pragma unroll
      for (int i = 0; i < MT_O; ++i) {
#pragma unroll
        for (int j = 0; j < MT_H; ++j) red[64 * (t++)] = dw_out[i][j];
        redb[64 * (u++)] = db_out[i];
      }
    }
    __syncthreads();
    if (wave == 0) {
      int t = 0, u = 0;
#pragma unroll
      for (int i = 0; i < MT_H; ++i) {
#pragma unroll
        for (int j = 0; j < MT_I; ++j) dw_in[i][j] += red[64 * (t++)];
        db_in[i] += redb[64 * (u++)];
#pragma unroll
        for (int k = 0; k < NH; ++k) {
          if (k < NREG) {
#pragma unroll
            for (int j = 0; j < MT_H; ++j) dw_hid[k < NREG ? k : 0][i][j] += red[64 * (t++)];
          }
          db_hid[k][i] += redb[64 * (u++)];
        }
      }
#pragma unroll
      for (int i = 0; i < MT_O; ++i) {
#pragma unroll
        for (int j = 0; j < MT_H; ++j) dw_out[i][j] += red[64 * (t++)];
        db_out[i] += redb[64 * (u++)];
      }
    }
    __syncthreads();
  }
  if (wave != 0) return;
#pragma unroll
  for (int i = 0; i < MT_H; ++i) {
#pragma unroll
    for (int j = 0; j < MT_I; ++j) flush_dw_tile(a.dw_in, a.d_hidden, a.d_in, i, j, lane, dw_in[i][j]);
    flush_db(a.db_in, a.d_hidden, i, lane, db_in[i]);
#pragma unroll
    for (int k = 0; k < NH; ++k) {
#pragma unroll
      for (int j = 0; j < MT_H; ++j) {
        f32x4_t v;
        if (k < NREG) {
          v = dw_hid[k < NREG ? k : 0][i][j];
        } else {  // wave 0's LDS tiles are the first of the four waves'
          constexpr int PER_WAVE = LA * MT_H * MT_H * 64;
          const int at = (((k - NREG) * MT_H + i) * MT_H + j) * 64 + lane;
          v = (lacc[at] + lacc[PER_WAVE + at]) + (lacc[2 * PER_WAVE + at] + lacc[3 * PER_WAVE + at]);
        }
        flush_dw_tile(a.dw_hid + k * hh, a.d_hidden, a.d_hidden, i, j, lane, v);
      }
      flush_db(a.db_hid ? a.db_hid + (size_t)k * a.d_hidden : nullptr, a.d_hidden, i, lane, db_hid[k][i]);
    }
  }
#pragma unroll
  for (int i = 0; i < MT_O; ++i) {
#pragma unroll
    for (int j = 0; j < MT_H; ++j) flush_dw_tile(a.dw_out, a.d_out, a.d_hidden, i, j, lane, dw_out[i][j]);
    flush_db(a.db_out, a.d_out, i, lane, db_out[i]);
  }
}

}  // namespace nf
