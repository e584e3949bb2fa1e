// Declarations shared by the fused-MLP translation units.
#pragma once

#include "mlp_tile.h"

namespace nf {

struct MlpArgs {
  const uint16_t* x;
  int64_t x_stride;
  uint16_t* y;
  int64_t y_stride;
  const uint16_t* dy;
  int64_t dy_stride;
  uint16_t* dx;
  int64_t dx_stride;
  const uint16_t *w_in, *b_in, *w_hid, *b_hid, *w_out, *b_out;
  float *dw_in, *db_in, *dw_hid, *db_hid, *dw_out, *db_out;
  int64_t rows;
  int d_in, d_hidden, d_out, depth, act;
  int x_vec, y_vec, dy_vec, dx_vec;
  int waves;  // waves per workgroup
  int in_act; // activation applied to x as it is loaded (x holds pre-activations of a layer in front); dx = d/dx of that
  int x_conv; // 0: x / dx stored like the weights; 1: stored as float16 (weights bfloat16); 2: stored as bfloat16 (weights float16)
  // eight-wave backward only: non-NULL = every workgroup stores its sums into partials + blockIdx.x * partial_stride
  // ([dw_in | dw_hid | dw_out | db_in | db_hid | db_out], float32) instead of adding them to dw_* / db_*
  float* partials;
  int64_t partial_stride;
};

constexpr int FRAG_ELEMS = 64 * 8;  // 16-bit elements per fragment (1 KiB)
constexpr int TPITCH = 40;          // 16-bit elements per feature row of a transposed 32-row panel (80 B)

// Fragment of 8 values stored in the other 16-bit type -> the compute type (what a cast kernel in front would do).
__device__ __forceinline__ Frag convert_frag(Frag f, int x_conv) {
  if (x_conv == 1) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f.w[i] = pack2<BF16>(unpack_lo<F16>(f.w[i]), unpack_hi<F16>(f.w[i]));
  } else if (x_conv == 2) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f.w[i] = pack2<F16>(unpack_lo<BF16>(f.w[i]), unpack_hi<BF16>(f.w[i]));
  }
  return f;
}

template <typename T>
__device__ __forceinline__ void stage_bias(float* dst, const uint16_t* b, int n_valid, int n_pad, int tid, int nthreads) {
  for (int i = tid; i < n_pad; i += nthreads) dst[i] = (b != nullptr && i < n_valid) ? T::to_f32(b[i]) : 0.0f;
}

// acc[nt][mt] = bias + W(frags) * in[nt][kc]; K chunks outermost, so that the products into one accumulator tile are
// 2 * MT instructions apart
template <typename T, int MT, int KC>
__device__ __forceinline__ void layer_mma(f32x4_t (&acc)[2][4], const Frag (&in)[2][2], const uint16_t* frags,
                                          const float* bias, int lane) {
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const f32x4_t b4 = *reinterpret_cast<const f32x4_t*>(bias + 16 * mt + 4 * (lane >> 4));
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

// Park an accumulator-layout tile (lane (n,g): features 16*mt + 4*g + r of row 16*nt + n) into a
// transposed panel panel[feature][row].
__device__ __forceinline__ void park_tile_T(uint16_t* panel, int mt, int nt, int lane, uint32_t p01, uint32_t p23) {
  const int n = (lane & 15) + 16 * nt;
  const int f = 16 * mt + 4 * (lane >> 4);
  panel[(f + 0) * TPITCH + n] = (uint16_t)(p01 & 0xffffu);
  panel[(f + 1) * TPITCH + n] = (uint16_t)(p01 >> 16);
  panel[(f + 2) * TPITCH + n] = (uint16_t)(p23 & 0xffffu);
  panel[(f + 3) * TPITCH + n] = (uint16_t)(p23 >> 16);
}
// Park a natural-order fragment (lane (n,g): features 32*kc + 8*g + j of row 16*nt + n).
__device__ __forceinline__ void park_frag_T(uint16_t* panel, int kc, int nt, int lane, const Frag& f) {
  const int n = (lane & 15) + 16 * nt;
  const int c = 32 * kc + 8 * (lane >> 4);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    panel[(c + 2 * j) * TPITCH + n] = (uint16_t)(f.w[j] & 0xffffu);
    panel[(c + 2 * j + 1) * TPITCH + n] = (uint16_t)(f.w[j] >> 16);
  }
}
// Operand of a K = 32-rows product: lane (i, g) reads rows 8*g .. 8*g+7 of feature 16*t + i.
__device__ __forceinline__ Frag panel_frag(const uint16_t* panel, int t, int lane) {
  Frag f;
  f.u = *reinterpret_cast<const uint4*>(panel + (16 * t + (lane & 15)) * TPITCH + 8 * (lane >> 4));
  return f;
}

// dW tile (mt over output features, nt over input features): lane (n, g) reg r is
// dW[16*mt + 4*g + r][16*nt + n].
// store: plain stores (the tile belongs to this workgroup alone) instead of atomic adds.
__device__ __forceinline__ void flush_dw_tile(float* dw, int out_dim, int in_dim, int mt, int nt, int lane, f32x4_t v,
                                              bool store = false) {
  const int c = 16 * nt + (lane & 15);
  const int r0 = 16 * mt + 4 * (lane >> 4);
  if (c >= in_dim) return;
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (r0 + r < out_dim) {
      if (store) dw[(size_t)(r0 + r) * in_dim + c] = v[r];
      else unsafeAtomicAdd(dw + (size_t)(r0 + r) * in_dim + c, v[r]);
    }
}

// Compute units of the current device.  The count is cached per device ordinal (written once with the same value by
// whichever thread asks first); besides the thread-local error text this is the only state the library keeps.
inline int device_cus() {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cus[dev] == 0) {
    hipDeviceProp_t p;
    int n = 0;
    if (hipGetDeviceProperties(&p, dev) == hipSuccess) n = p.multiProcessorCount;
    cus[dev] = n > 0 ? n : 256;
  }
  return cus[dev];
}

constexpr size_t LDS_LIMIT = 160 * 1024;


// Specialised backward for exactly one hidden layer (fused_mlp_bwd2.hip), bias gradients included.
// *handled = false: shape not covered, nothing was launched.
int launch_mlp_bwd2(const MlpArgs& a, int dtype, hipStream_t s, bool* handled);
// The same for two or three hidden-to-hidden layers of width 64 with ReLU (fused_mlp_bwdn.hip).
int launch_mlp_bwdn(const MlpArgs& a, int dtype, hipStream_t s, bool* handled);
// The benchmark shape of launch_mlp_bwd2 (d_in <= 32, d_hidden = 64, d_out <= 16, ReLU, aligned rows, extents below
// 2^31 bytes) on eight waves per workgroup (fused_mlp_bwd2_w8.hip).  *handled = false: not that shape.
int launch_mlp_bwd2_w8(const MlpArgs& a, int dtype, hipStream_t s, bool* handled);
// The same with the weight and bias gradients summed in a fixed order and written, rounded to `dtype`, into out[6]
// (dw_in, db_in, dw_hid, db_hid, dw_out, db_out; NULL entries skipped); workspace: mlp_bwd2_w8_rounded_bytes().
// Also covers the shapes of launch_mlp_bwd2_ws.
size_t mlp_bwd2_w8_rounded_bytes(int d_in, int d_hidden, int d_out);
int launch_mlp_bwd2_w8_rounded(const MlpArgs& a, int dtype, void* const out[6], void* workspace, hipStream_t s, bool* handled);


// One hidden layer, width 64, ReLU, with d_in > 32 or d_out > 16 (aligned rows, extents below 2^31 bytes): chain and
// gradient waves (fused_mlp_bwd2_ws.hip).  *handled = false: not such a call, nothing was launched.
int launch_mlp_bwd2_ws(const MlpArgs& a, int dtype, hipStream_t s, bool* handled, int* blocks_out = nullptr);

// The forward of one-hidden-layer ReLU networks of width 64 with aligned rows (fused_mlp_fwd2.hip).  *handled = false: not that shape, nothing was launched.
int launch_mlp_fwd2(const MlpArgs& a, int dtype, hipStream_t s, bool* handled);

// float32 storage and float32 products (fused_mlp_f32.hip).  The backward needs mlp32_bwd_workspace_bytes of scratch.
size_t mlp32_bwd_workspace_bytes(int64_t rows, int d_hidden, int depth);
int mlp32_fwd(const float* x, int64_t x_stride, float* y, int64_t y_stride, const float* w_in, const float* b_in,
              const float* w_hid, const float* b_hid, const float* w_out, const float* b_out, int64_t rows, int d_in,
              int d_hidden, int d_out, int depth, int act, hipStream_t s);
int mlp32_bwd(const float* x, int64_t x_stride, const float* dy, int64_t dy_stride, float* dx, int64_t dx_stride,
              const float* w_in, const float* b_in, const float* w_hid, const float* b_hid, const float* w_out, float* dw_in,
              float* db_in, float* dw_hid, float* db_hid, float* dw_out, float* db_out, int64_t rows, int d_in, int d_hidden,
              int d_out, int depth, int act, void* workspace, int64_t workspace_bytes, hipStream_t s);

}  // namespace nf
