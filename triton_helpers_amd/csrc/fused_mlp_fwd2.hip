// The forward of one-hidden-layer ReLU networks of width 64 (d_in <= 64, d_out <= 64; the decoder / benchmark shape
// 32 -> 64 -> 64 -> 16 and the 64-wide shapes of the reference's own benchmark), 8-byte aligned rows, as a kernel of
// its own per (input, output) width class: twelve waves per workgroup, the chunk body one basic block (no
// run-time tests of activation, depth, alignment or row count inside it), rows addressed through buffer descriptors
// (reads past the end return zero, stores past it are dropped), the next chunk's rows requested before this one's
// products.  Everything else stays on mlp_fwd_k (fused_mlp.hip), which loops over a run-time depth.
#include "fused_mlp_bwd2_kernels.h"

namespace nf {

// Workgroups per CU of the launch (15 KB of LDS and under 128 registers each: the grid, not the chip, sets it).
#ifndef NF_FWD2_WG_PER_CU
#define NF_FWD2_WG_PER_CU 1
#endif

#ifndef NF_FWD2_WAVES
#define NF_FWD2_WAVES 12
#endif

// XC: how x is stored (MlpArgs::x_conv); KIN / OUTP: d_in / d_out rounded up to 32 or 64 / 16 or 64.
// Twelve waves where the weight fragments (held in registers across chunks) leave room for three waves per SIMD,
// eight for the 64-wide inputs / outputs.
constexpr int fwd2_waves(int kin, int outp) { return (kin == 32 && outp == 16) ? NF_FWD2_WAVES : 8; }

template <typename T, int XC, int KIN = 32, int OUTP = 16>
__global__ __launch_bounds__(64 * fwd2_waves(KIN, OUTP)) void mlp_fwd2_k(MlpArgs a) {
  constexpr int HP = 64, NT = 2, WAVES = fwd2_waves(KIN, OUTP);
  constexpr int KC_IN = KIN / 32, KC_H = HP / 32, MT_H = HP / 16, MT_O = OUTP / 16;
  constexpr int ROWS = 16 * NT;
  constexpr int nthreads = 64 * WAVES;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t n_chunks = (a.rows + ROWS - 1) / ROWS;
  const int64_t wave_stride = (int64_t)gridDim.x * WAVES;
  const int64_t first_chunk = (int64_t)blockIdx.x * WAVES + wave;
  const __amdgpu_buffer_rsrc_t rs_x = rows_rsrc(a.x, a.rows, a.x_stride), rs_y = rows_rsrc(a.y, a.rows, a.y_stride);
  uint32_t off_x[KC_IN][2];
#pragma unroll
  for (int kc = 0; kc < KC_IN; ++kc)
#pragma unroll
    for (int h = 0; h < 2; ++h) off_x[kc][h] = piece_offset(lane & 15, 32 * kc + 16 * h + 4 * (lane >> 4), a.d_in, a.x_stride);
  uint32_t off_y[MT_O];
#pragma unroll
  for (int mt = 0; mt < MT_O; ++mt) off_y[mt] = piece_offset(lane & 15, 16 * mt + 4 * (lane >> 4), a.d_out, a.y_stride);
  auto load_x = [&](int64_t chunk, int nt, int kc) {
    const uint32_t at = (uint32_t)((chunk * ROWS + 16 * nt) * a.x_stride * 2);
    const buf_v2u lo = __builtin_amdgcn_raw_buffer_load_b64(rs_x, off_x[kc][0] + at, 0, 0);
    const buf_v2u hi = __builtin_amdgcn_raw_buffer_load_b64(rs_x, off_x[kc][1] + at, 0, 0);
    Frag f;
    f.w[0] = lo[0]; f.w[1] = lo[1]; f.w[2] = hi[0]; f.w[3] = hi[1];
    return f;
  };
  // rows in flight per wave: the next chunk, and for 64-wide inputs (eight waves, 4 KB per chunk) the one behind it too (64 -> 64 -> 16: 45.8 -> 40.9 us per 2^20 rows)
  constexpr bool DEEP = KIN > 32;
  Frag nx[NT][KC_IN], nnx[NT][KC_IN];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int kc = 0; kc < KC_IN; ++kc) {
      nx[nt][kc] = load_x(first_chunk, nt, kc);
      if constexpr (DEEP) nnx[nt][kc] = load_x(first_chunk + wave_stride, nt, kc);
    }

  uint16_t* f_in = reinterpret_cast<uint16_t*>(smem);   // W_in  [MT_H][KC_IN]
  uint16_t* f_hid = f_in + MT_H * KC_IN * FRAG_ELEMS;   // W_hid [MT_H][KC_H]
  uint16_t* f_out = f_hid + MT_H * KC_H * FRAG_ELEMS;   // W_out [MT_O][KC_H]
  float* bias_in = reinterpret_cast<float*>(f_out + MT_O * KC_H * FRAG_ELEMS);
  float* bias_hid = bias_in + HP;
  float* bias_out = bias_hid + HP;
  stage_weight_frags<true, false, nthreads>(f_in, a.w_in, a.d_hidden, a.d_in, MT_H, KC_IN, tid, nthreads);
  stage_weight_frags<true, false, nthreads>(f_hid, a.w_hid, a.d_hidden, a.d_hidden, MT_H, KC_H, tid, nthreads);
  stage_weight_frags<true, false, nthreads>(f_out, a.w_out, a.d_out, a.d_hidden, MT_O, KC_H, tid, nthreads);
  stage_bias<T>(bias_in, a.b_in, a.d_hidden, HP, tid, nthreads);
  stage_bias<T>(bias_hid, a.b_hid, a.d_hidden, HP, tid, nthreads);
  stage_bias<T>(bias_out, a.b_out, a.d_out, OUTP, tid, nthreads);
  __syncthreads();

  for (int64_t chunk = first_chunk; chunk < n_chunks; chunk += wave_stride) {
    Frag in[NT][2], h[NT][2];
    f32x4_t acc[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int kc = 0; kc < KC_IN; ++kc) {
        in[nt][kc] = XC == 0 ? nx[nt][kc] : convert_frag(nx[nt][kc], XC);
        if constexpr (DEEP) {
          nx[nt][kc] = nnx[nt][kc];
          nnx[nt][kc] = load_x(chunk + 2 * wave_stride, nt, kc);
        } else {
          nx[nt][kc] = load_x(chunk + wave_stride, nt, kc);
        }
      }
    layer_nt<T, NT, MT_H, KC_IN, 1>(acc, in, f_in, bias_in, lane);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT_H; ++mt) {
        h[nt][mt >> 1].w[2 * (mt & 1)] = relu_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]));
        h[nt][mt >> 1].w[2 * (mt & 1) + 1] = relu_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]));
      }
    layer_nt<T, NT, MT_H, KC_H, 1>(acc, h, f_hid, bias_hid, lane);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT_H; ++mt) {
        h[nt][mt >> 1].w[2 * (mt & 1)] = relu_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]));
        h[nt][mt >> 1].w[2 * (mt & 1) + 1] = relu_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]));
      }
    layer_nt<T, NT, MT_O, KC_H, 1>(acc, h, f_out, bias_out, lane);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT_O; ++mt) {
        buf_v2u o;
        o[0] = pack2<T>(acc[nt][mt][0], acc[nt][mt][1]);
        o[1] = pack2<T>(acc[nt][mt][2], acc[nt][mt][3]);
        __builtin_amdgcn_raw_buffer_store_b64(o, rs_y, off_y[mt] + (uint32_t)((chunk * ROWS + 16 * nt) * a.y_stride * 2), 0, 0);
      }
  }
}

template <typename T, int KIN, int OUTP>
static int launch_fwd2(const MlpArgs& a0, hipStream_t s) {
  MlpArgs a = a0;
  constexpr int WAVES = fwd2_waves(KIN, OUTP), ROWS = 32;
  constexpr size_t LDS = ((size_t)4 * (KIN / 32) + 4 * 2 + (OUTP / 16) * 2) * 1024 + (size_t)(64 + 64 + OUTP) * 4;
  a.waves = WAVES;
  const int64_t chunks = (a.rows + ROWS - 1) / ROWS;
  int64_t blocks = (chunks + WAVES - 1) / WAVES;
  const int64_t cap = (int64_t)device_cus() * NF_FWD2_WG_PER_CU;
  if (blocks > cap) blocks = cap;
  constexpr int XC_OTHER = T::code == NF_BF16 ? 1 : 2;
  const void* kern = a.x_conv == 0 ? (const void*)mlp_fwd2_k<T, 0, KIN, OUTP> : (const void*)mlp_fwd2_k<T, XC_OTHER, KIN, OUTP>;
  void* args[] = {(void*)&a};
  const hipError_t e = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(64 * WAVES), args, LDS, s);
  if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(mlp_fwd2): %s", hipGetErrorString(e));
  return check_launch("mlp_fwd2");
}

int launch_mlp_fwd2(const MlpArgs& a, int dtype, hipStream_t s, bool* handled) {
  *handled = false;
  const int xc_other = dtype == NF_BF16 ? 1 : 2;
  const auto rows8 = [](const void* p, int64_t stride) { return (uintptr_t)p % 8 == 0 && stride % 4 == 0; };
  const bool shape = a.depth == 2 && a.d_hidden == 64 && a.d_in <= 64 && a.d_out <= 64 && a.act == NF_ACT_RELU && a.in_act == NF_ACT_NONE &&
                     (a.x_conv == 0 || a.x_conv == xc_other);
  const bool aligned = a.d_in % 4 == 0 && a.d_out % 4 == 0 && rows8(a.x, a.x_stride) && rows8(a.y, a.y_stride);
  const bool in_reach = rows_in_reach(a.rows, a.x_stride) && rows_in_reach(a.rows, a.y_stride);
  if (!shape || !aligned || !in_reach) return 0;
  *handled = true;
  const bool wide_in = a.d_in > 32, wide_out = a.d_out > 16;
#define NF_FWD2_DISPATCH(T)                                          \
  (wide_in ? (wide_out ? launch_fwd2<T, 64, 64>(a, s) : launch_fwd2<T, 64, 16>(a, s)) \
           : (wide_out ? launch_fwd2<T, 32, 64>(a, s) : launch_fwd2<T, 32, 16>(a, s)))
  return dtype == NF_BF16 ? NF_FWD2_DISPATCH(BF16) : NF_FWD2_DISPATCH(F16);
#undef NF_FWD2_DISPATCH
}

}  // namespace nf
