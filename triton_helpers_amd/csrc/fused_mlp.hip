// Fully fused MLP for gfx950: forward and backward, 16-bit storage (bf16 / fp16),
// float32 accumulation on v_mfma_f32_16x16x32.
//
// Layer math follows triton_helpers/layers/fully_fused_mlp/kernel.py:17-74 of the reference:
//   z = x W^T + b (float32 accumulate), h = act(z) rounded to the storage type, no activation
//   after the output layer; backward dz = act'(z) * dh, dW = dz^T h_prev, dh_prev = dz W.
//
// Forward: weights are staged once per workgroup into LDS as MFMA A fragments; each wave
// walks 32-row chunks and keeps every activation in registers (see mlp_tile.h).
// Backward: the forward is recomputed once per chunk from x; each layer's input is parked
// in LDS transposed ([feature][row]) so that dW = dZ^T H can read both operands as
// K = 32 data rows; act'(z) is parked as a register image.  Weight gradients accumulate in
// float32 registers over the wave's whole row loop (up to REG_HIDDEN hidden layers), are
// reduced across the workgroup through LDS and leave with one coalesced atomic add per
// 64-byte segment; deeper nets add the hidden-layer partials to memory chunk by chunk.
#include <vector>

#include "fused_mlp.h"

namespace nf {

// activation + rounding of a hidden layer; the packed tiles become the next layer's B fragments
template <typename T, int KC_H, bool RELU>
__device__ __forceinline__ void hidden_epilogue(const f32x4_t (&acc)[2][4], Frag (&in)[2][2], int act) {
  with_act(RELU ? NF_ACT_RELU : act, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int kc = 0; kc < KC_H; ++kc) {
        act_pack<T, RELU>(acc[nt][2 * kc], ACT, in[nt][kc].w[0], in[nt][kc].w[1]);
        act_pack<T, RELU>(acc[nt][2 * kc + 1], ACT, in[nt][kc].w[2], in[nt][kc].w[3]);
      }
  });
}

// ---------------------------------------------------------------------------------------
// Forward
// ---------------------------------------------------------------------------------------
// XC: how x is stored (MlpArgs::x_conv), fixed at compile time.
template <typename T, int KIN, int HP, int OUTP, int XC>
__global__ __launch_bounds__(512) void mlp_fwd_k(MlpArgs a) {
  constexpr int KC_IN = KIN / 32, KC_H = HP / 32, MT_H = HP / 16, MT_O = OUTP / 16;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n_hid = a.depth - 1;

  uint16_t* f_in = reinterpret_cast<uint16_t*>(smem);
  uint16_t* f_hid = f_in + MT_H * KC_IN * FRAG_ELEMS;
  uint16_t* f_out = f_hid + (size_t)n_hid * MT_H * KC_H * FRAG_ELEMS;
  float* bias_in = reinterpret_cast<float*>(f_out + MT_O * KC_H * FRAG_ELEMS);
  float* bias_hid = bias_in + HP;
  float* bias_out = bias_hid + (size_t)n_hid * HP;

  stage_weight_frags<false, false>(f_in, a.w_in, a.d_hidden, a.d_in, MT_H, KC_IN, tid, nthreads);
  for (int k = 0; k < n_hid; ++k)
    stage_weight_frags<true, false>(f_hid + (size_t)k * MT_H * KC_H * FRAG_ELEMS,
                                    a.w_hid + (size_t)k * a.d_hidden * a.d_hidden, a.d_hidden, a.d_hidden, MT_H, KC_H,
                                    tid, nthreads);
  stage_weight_frags<true, false>(f_out, a.w_out, a.d_out, a.d_hidden, MT_O, KC_H, tid, nthreads);
  stage_bias<T>(bias_in, a.b_in, a.d_hidden, HP, tid, nthreads);
  for (int k = 0; k < n_hid; ++k)
    stage_bias<T>(bias_hid + k * HP, a.b_hid ? a.b_hid + (size_t)k * a.d_hidden : nullptr, a.d_hidden, HP, tid, nthreads);
  stage_bias<T>(bias_out, a.b_out, a.d_out, OUTP, tid, nthreads);
  __syncthreads();

  const bool relu = a.act == NF_ACT_RELU;
  const int64_t n_chunks = (a.rows + 31) / 32;
  const int64_t wave_stride = (int64_t)gridDim.x * a.waves;
  // the next chunk's rows are requested before the current chunk is computed (loads past the end return zeros)
  Frag nxt[2][2];
  const int64_t first_chunk = (int64_t)blockIdx.x * a.waves + wave;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int kc = 0; kc < KC_IN; ++kc)
      nxt[nt][kc] = load_rows_frag(a.x, a.x_stride, first_chunk * 32 + 16 * nt, a.rows, a.d_in, kc, lane, a.x_vec);
  for (int64_t chunk = first_chunk; chunk < n_chunks; chunk += wave_stride) {
    const int64_t row0 = chunk * 32;
    Frag in[2][2];
    f32x4_t acc[2][4];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int kc = 0; kc < KC_IN; ++kc) {
        in[nt][kc] = XC == 0 ? nxt[nt][kc] : convert_frag(nxt[nt][kc], XC);
        if (a.in_act != NF_ACT_NONE) in[nt][kc] = act_frag<T>(in[nt][kc], a.in_act);
        nxt[nt][kc] = load_rows_frag(a.x, a.x_stride, (chunk + wave_stride) * 32 + 16 * nt, a.rows, a.d_in, kc, lane, a.x_vec);
      }

    layer_mma<T, MT_H, KC_IN>(acc, in, f_in, bias_in, lane);
    if (relu)
      hidden_epilogue<T, KC_H, true>(acc, in, a.act);
    else
      hidden_epilogue<T, KC_H, false>(acc, in, a.act);
    for (int k = 0; k < n_hid; ++k) {
      layer_mma<T, MT_H, KC_H>(acc, in, f_hid + (size_t)k * MT_H * KC_H * FRAG_ELEMS, bias_hid + k * HP, lane);
      if (relu)
        hidden_epilogue<T, KC_H, true>(acc, in, a.act);
      else
        hidden_epilogue<T, KC_H, false>(acc, in, a.act);
    }
    layer_mma<T, MT_O, KC_H>(acc, in, f_out, bias_out, lane);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT_O; ++mt)
        store_rows_tile<T>(a.y, a.y_stride, row0 + 16 * nt, a.rows, a.d_out, mt, lane, acc[nt][mt], a.y_vec);
  }
}

// ---------------------------------------------------------------------------------------
// Backward
// ---------------------------------------------------------------------------------------
// forward recompute of one layer inside the backward: activation, park h^T, park the gate image
template <typename T, int MT_H, bool RELU>
__device__ __forceinline__ void recompute_epilogue(const f32x4_t (&acc)[2][4], Frag (&in)[2][2], uint16_t* panel, uint32_t* im,
                                                   int act, int lane) {
  with_act(RELU ? NF_ACT_RELU : act, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT_H; ++mt) {
        uint32_t h01, h23, g01, g23;
        act_pack<T, RELU>(acc[nt][mt], ACT, h01, h23);
        gate_pack<T, RELU>(acc[nt][mt], ACT, h01, h23, g01, g23);
        in[nt][mt >> 1].w[2 * (mt & 1)] = h01;
        in[nt][mt >> 1].w[2 * (mt & 1) + 1] = h23;
        park_tile_T(panel, mt, nt, lane, h01, h23);
        im[((mt * 2 + nt) * 2 + 0) * 64 + lane] = g01;
        im[((mt * 2 + nt) * 2 + 1) * 64 + lane] = g23;
      }
  });
}

template <typename T, int KIN, int HP, int OUTP, int REG_HIDDEN>
__global__ __launch_bounds__(256) void mlp_bwd_k(MlpArgs a) {
  constexpr int KC_IN = KIN / 32, KC_H = HP / 32, MT_H = HP / 16, MT_I = KIN / 16, MT_O = OUTP / 16;
  constexpr int KC_O = (OUTP + 31) / 32;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n_hid = a.depth - 1;
  const bool regs_hold_hidden = n_hid <= REG_HIDDEN;

  // ---- LDS carve-up: weights (forward + transposed), biases, then per-wave panels ----
  uint16_t* f_in = reinterpret_cast<uint16_t*>(smem);                            // [MT_H][KC_IN]
  uint16_t* f_hid = f_in + MT_H * KC_IN * FRAG_ELEMS;                            // [n_hid][MT_H][KC_H]
  uint16_t* t_in = f_hid + (size_t)n_hid * MT_H * KC_H * FRAG_ELEMS;             // W_in^T  [MT_I][KC_H]
  uint16_t* t_hid = t_in + MT_I * KC_H * FRAG_ELEMS;                             // W_hid^T [n_hid][MT_H][KC_H]
  uint16_t* t_out = t_hid + (size_t)n_hid * MT_H * KC_H * FRAG_ELEMS;            // W_out^T [MT_H][KC_O]
  float* bias_in = reinterpret_cast<float*>(t_out + MT_H * KC_O * FRAG_ELEMS);   // [HP]
  float* bias_hid = bias_in + HP;                                                // [n_hid][HP]
  uint16_t* wave_base = reinterpret_cast<uint16_t*>(bias_hid + (size_t)n_hid * HP);
  // per wave: x^T [KIN], h_k^T [depth][HP], dz^T [max(HP,OUTP32)], act' images [depth][MT_H*2*2*64 dwords]
  constexpr int DZ_FEATS = HP > 32 * KC_O ? HP : 32 * KC_O;
  const size_t panel_elems = (size_t)(KIN + (size_t)a.depth * HP + DZ_FEATS) * TPITCH;
  const size_t image_elems = (size_t)a.depth * MT_H * 2 * 2 * 64 * 2;  // in 16-bit units
  const size_t per_wave = panel_elems + image_elems;
  uint16_t* xT = wave_base + (size_t)wave * per_wave;
  uint16_t* hT = xT + KIN * TPITCH;                   // hT + (k-1)*HP*TPITCH : h_k^T, k = 1..depth
  uint16_t* dzT = hT + (size_t)a.depth * HP * TPITCH;
  uint32_t* img = reinterpret_cast<uint32_t*>(dzT + DZ_FEATS * TPITCH);  // [depth][MT_H][2 nt][2][64]

  stage_weight_frags<false, false>(f_in, a.w_in, a.d_hidden, a.d_in, MT_H, KC_IN, tid, nthreads);
  stage_weight_frags<true, true>(t_in, a.w_in, a.d_hidden, a.d_in, MT_I, KC_H, tid, nthreads);
  for (int k = 0; k < n_hid; ++k) {
    const uint16_t* w = a.w_hid + (size_t)k * a.d_hidden * a.d_hidden;
    stage_weight_frags<true, false>(f_hid + (size_t)k * MT_H * KC_H * FRAG_ELEMS, w, a.d_hidden, a.d_hidden, MT_H, KC_H, tid, nthreads);
    stage_weight_frags<true, true>(t_hid + (size_t)k * MT_H * KC_H * FRAG_ELEMS, w, a.d_hidden, a.d_hidden, MT_H, KC_H, tid, nthreads);
  }
  stage_weight_frags<false, true>(t_out, a.w_out, a.d_out, a.d_hidden, MT_H, KC_O, tid, nthreads);
  stage_bias<T>(bias_in, a.b_in, a.d_hidden, HP, tid, nthreads);
  for (int k = 0; k < n_hid; ++k)
    stage_bias<T>(bias_hid + k * HP, a.b_hid ? a.b_hid + (size_t)k * a.d_hidden : nullptr, a.d_hidden, HP, tid, nthreads);
  // zero the padding rows of the dz panel once (features >= what a layer writes are read as zero operands)
  for (int i = lane; i < DZ_FEATS * TPITCH; i += 64) dzT[i] = 0;
  __syncthreads();

  f32x4_t dw_in[MT_H][MT_I];
  f32x4_t dw_out[MT_O][MT_H];
  f32x4_t dw_hid[REG_HIDDEN > 0 ? REG_HIDDEN : 1][MT_H][MT_H];
  f32x4_t db_acc_in[MT_H], db_acc_hid[REG_HIDDEN > 0 ? REG_HIDDEN : 1][MT_H];
  const f32x4_t zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int i = 0; i < MT_H; ++i) {
    db_acc_in[i] = zero4;
#pragma unroll
    for (int j = 0; j < MT_I; ++j) dw_in[i][j] = zero4;
  }
#pragma unroll
  for (int i = 0; i < MT_O; ++i)
#pragma unroll
    for (int j = 0; j < MT_H; ++j) dw_out[i][j] = zero4;
#pragma unroll
  for (int h = 0; h < (REG_HIDDEN > 0 ? REG_HIDDEN : 1); ++h)
#pragma unroll
    for (int i = 0; i < MT_H; ++i) {
      db_acc_hid[h][i] = zero4;
#pragma unroll
      for (int j = 0; j < MT_H; ++j) dw_hid[h][i][j] = zero4;
    }
  const bool want_db = a.db_in != nullptr || a.db_hid != nullptr;  // db_out is a separate pass over dy
  const bool relu = a.act == NF_ACT_RELU;

  const int64_t n_chunks = (a.rows + 31) / 32;
  const int64_t wave_stride = (int64_t)gridDim.x * a.waves;
  // the next chunk's x and dy rows are requested before the current chunk is computed
  Frag nx[2][2], ndy[2][2];
  const int64_t first_chunk = (int64_t)blockIdx.x * a.waves + wave;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
    for (int kc = 0; kc < KC_IN; ++kc)
      nx[nt][kc] = load_rows_frag(a.x, a.x_stride, first_chunk * 32 + 16 * nt, a.rows, a.d_in, kc, lane, a.x_vec);
#pragma unroll
    for (int kc = 0; kc < KC_O; ++kc)
      ndy[nt][kc] = load_rows_frag(a.dy, a.dy_stride, first_chunk * 32 + 16 * nt, a.rows, a.d_out, kc, lane, a.dy_vec);
  }
  for (int64_t chunk = first_chunk; chunk < n_chunks; chunk += wave_stride) {
    const int64_t row0 = chunk * 32;
    Frag in[2][2];
    f32x4_t acc[2][4];
    Frag dz[2][2];

    // ---------------- forward recompute; park inputs (transposed) and act'(z) ----------------
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int kc = 0; kc < KC_IN; ++kc) {
        in[nt][kc] = nx[nt][kc];
        if (a.in_act != NF_ACT_NONE) in[nt][kc] = act_frag<T>(in[nt][kc], a.in_act);
        nx[nt][kc] = load_rows_frag(a.x, a.x_stride, (chunk + wave_stride) * 32 + 16 * nt, a.rows, a.d_in, kc, lane, a.x_vec);
        park_frag_T(xT, kc, nt, lane, in[nt][kc]);
      }
#pragma unroll
      for (int kc = 0; kc < KC_O; ++kc) {
        dz[nt][kc] = ndy[nt][kc];
        ndy[nt][kc] = load_rows_frag(a.dy, a.dy_stride, (chunk + wave_stride) * 32 + 16 * nt, a.rows, a.d_out, kc, lane, a.dy_vec);
      }
    }
    for (int k = 1; k <= a.depth; ++k) {
      if (k == 1)
        layer_mma<T, MT_H, KC_IN>(acc, in, f_in, bias_in, lane);
      else
        layer_mma<T, MT_H, KC_H>(acc, in, f_hid + (size_t)(k - 2) * MT_H * KC_H * FRAG_ELEMS, bias_hid + (k - 2) * HP, lane);
      uint16_t* panel = hT + (size_t)(k - 1) * HP * TPITCH;
      uint32_t* im = img + (size_t)(k - 1) * MT_H * 2 * 2 * 64;
      if (relu)
        recompute_epilogue<T, MT_H, true>(acc, in, panel, im, a.act, lane);
      else
        recompute_epilogue<T, MT_H, false>(acc, in, panel, im, a.act, lane);
    }

    // ---------------- output layer: dz_out = dy ----------------
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int kc = 0; kc < KC_O; ++kc) park_frag_T(dzT, kc, nt, lane, dz[nt][kc]);
    {
      const uint16_t* hprev = hT + (size_t)(a.depth - 1) * HP * TPITCH;
      Frag hb[MT_H];
#pragma unroll
      for (int j = 0; j < MT_H; ++j) hb[j] = panel_frag(hprev, j, lane);
#pragma unroll
      for (int i = 0; i < MT_O; ++i) {
        const Frag da = panel_frag(dzT, i, lane);
#pragma unroll
        for (int j = 0; j < MT_H; ++j) dw_out[i][j] = mfma16<T>(da, hb[j], dw_out[i][j]);
      }
      // dh_depth = W_out^T dy
#pragma unroll
      for (int mt = 0; mt < MT_H; ++mt) {
        acc[0][mt] = zero4;
        acc[1][mt] = zero4;
#pragma unroll
        for (int kc = 0; kc < KC_O; ++kc) {
          const Frag wa = lds_frag(t_out, mt * KC_O + kc, lane);
          acc[0][mt] = mfma16<T>(wa, dz[0][kc], acc[0][mt]);
          acc[1][mt] = mfma16<T>(wa, dz[1][kc], acc[1][mt]);
        }
      }
    }

    // ---------------- hidden layers (k = depth .. 2) and the input layer (k = 1) ----------------
    for (int k = a.depth; k >= 1; --k) {
      // dz_k = dh_k * act'(z_k), rounded to the storage type; park transposed
      const uint32_t* im = img + (size_t)(k - 1) * MT_H * 2 * 2 * 64;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT_H; ++mt) {
          const uint32_t g01 = im[((mt * 2 + nt) * 2 + 0) * 64 + lane];
          const uint32_t g23 = im[((mt * 2 + nt) * 2 + 1) * 64 + lane];
          uint32_t p01, p23;
          if (relu)
            gate_apply<T, true>(acc[nt][mt], g01, g23, p01, p23);
          else
            gate_apply<T, false>(acc[nt][mt], g01, g23, p01, p23);
          dz[nt][mt >> 1].w[2 * (mt & 1)] = p01;
          dz[nt][mt >> 1].w[2 * (mt & 1) + 1] = p23;
          park_tile_T(dzT, mt, nt, lane, p01, p23);
          if (want_db) {
            const f32x4_t dzv = {unpack_lo<T>(p01), unpack_hi<T>(p01), unpack_lo<T>(p23), unpack_hi<T>(p23)};
            if (k == 1) {
              db_acc_in[mt] += dzv;
            } else if (regs_hold_hidden) {
#pragma unroll
              for (int h = 0; h < REG_HIDDEN; ++h)
                if (h == k - 2) db_acc_hid[h][mt] += dzv;
            } else if (a.db_hid != nullptr) {
              // deep nets: fold the 16 rows of this tile now and add to memory
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                float t = dzv[r];
                t += __shfl_xor(t, 1);
                t += __shfl_xor(t, 2);
                t += __shfl_xor(t, 4);
                t += __shfl_xor(t, 8);
                const int f = 16 * mt + 4 * (lane >> 4) + r;
                if ((lane & 15) == 0 && f < a.d_hidden) unsafeAtomicAdd(a.db_hid + (size_t)(k - 2) * a.d_hidden + f, t);
              }
            }
          }
        }
      if (k == 1) {
        // dW_in += dz_1^T x ; dx = W_in^T dz_1
        Frag xb[MT_I];
#pragma unroll
        for (int j = 0; j < MT_I; ++j) xb[j] = panel_frag(xT, j, lane);
#pragma unroll
        for (int i = 0; i < MT_H; ++i) {
          const Frag da = panel_frag(dzT, i, lane);
#pragma unroll
          for (int j = 0; j < MT_I; ++j) dw_in[i][j] = mfma16<T>(da, xb[j], dw_in[i][j]);
        }
        if (a.dx != nullptr) {
#pragma unroll
          for (int mt = 0; mt < MT_I; ++mt) {
            f32x4_t o0 = zero4, o1 = zero4;
#pragma unroll
            for (int kc = 0; kc < KC_H; ++kc) {
              const Frag wa = lds_frag(t_in, mt * KC_H + kc, lane);
              o0 = mfma16<T>(wa, dz[0][kc], o0);
              o1 = mfma16<T>(wa, dz[1][kc], o1);
            }
            if (a.in_act != NF_ACT_NONE) {
              // the stored x of these positions (just read by this wave: a cache hit) gives act'(x)
              const uint2 x0 = load_rows_tile(a.x, a.x_stride, row0, a.rows, a.d_in, mt, lane, a.x_vec != 0);
              const uint2 x1 = load_rows_tile(a.x, a.x_stride, row0 + 16, a.rows, a.d_in, mt, lane, a.x_vec != 0);
              o0 = input_gate<T>(o0, x0.x, x0.y, a.in_act);
              o1 = input_gate<T>(o1, x1.x, x1.y, a.in_act);
            }
            store_rows_tile<T>(a.dx, a.dx_stride, row0, a.rows, a.d_in, mt, lane, o0, a.dx_vec);
            store_rows_tile<T>(a.dx, a.dx_stride, row0 + 16, a.rows, a.d_in, mt, lane, o1, a.dx_vec);
          }
        }
      } else {
        // hidden layer k-2: dW += dz_k^T h_{k-1} ; dh_{k-1} = W^T dz_k
        const uint16_t* hprev = hT + (size_t)(k - 2) * HP * TPITCH;
        Frag hb[MT_H];
#pragma unroll
        for (int j = 0; j < MT_H; ++j) hb[j] = panel_frag(hprev, j, lane);
        if (regs_hold_hidden) {
#pragma unroll
          for (int h = 0; h < REG_HIDDEN; ++h)
            if (h == k - 2) {
#pragma unroll
              for (int i = 0; i < MT_H; ++i) {
                const Frag da = panel_frag(dzT, i, lane);
#pragma unroll
                for (int j = 0; j < MT_H; ++j) dw_hid[h][i][j] = mfma16<T>(da, hb[j], dw_hid[h][i][j]);
              }
            }
        } else {
          float* dst = a.dw_hid + (size_t)(k - 2) * a.d_hidden * a.d_hidden;
#pragma unroll
          for (int i = 0; i < MT_H; ++i) {
            const Frag da = panel_frag(dzT, i, lane);
#pragma unroll
            for (int j = 0; j < MT_H; ++j)
              flush_dw_tile(dst, a.d_hidden, a.d_hidden, i, j, lane, mfma16<T>(da, hb[j], zero4));
          }
        }
        const uint16_t* wt = t_hid + (size_t)(k - 2) * MT_H * KC_H * FRAG_ELEMS;
#pragma unroll
        for (int mt = 0; mt < MT_H; ++mt) {
          f32x4_t o0 = zero4, o1 = zero4;
#pragma unroll
          for (int kc = 0; kc < KC_H; ++kc) {
            const Frag wa = lds_frag(wt, mt * KC_H + kc, lane);
            o0 = mfma16<T>(wa, dz[0][kc], o0);
            o1 = mfma16<T>(wa, dz[1][kc], o1);
          }
          acc[0][mt] = o0;
          acc[1][mt] = o1;
        }
      }
    }
  }

  // ---------------- reduce the weight gradients over the workgroup, then one atomic pass ----------------
  // Reuse the (now idle) per-wave region as a float staging buffer, one wave at a time.
  __syncthreads();
  float* red = reinterpret_cast<float*>(wave_base);
  for (int w = 1; w < a.waves; ++w) {
    if (wave == w) {
      int t = 0;
#pragma unroll
      for (int i = 0; i < MT_H; ++i)
#pragma unroll
        for (int j = 0; j < MT_I; ++j) *reinterpret_cast<f32x4_t*>(red + ((t++) * 64 + lane) * 4) = dw_in[i][j];
#pragma unroll
      for (int i = 0; i < MT_O; ++i)
#pragma unroll
        for (int j = 0; j < MT_H; ++j) *reinterpret_cast<f32x4_t*>(red + ((t++) * 64 + lane) * 4) = dw_out[i][j];
#pragma unroll
      for (int h = 0; h < (REG_HIDDEN > 0 ? REG_HIDDEN : 1); ++h)
#pragma unroll
        for (int i = 0; i < MT_H; ++i)
#pragma unroll
          for (int j = 0; j < MT_H; ++j) *reinterpret_cast<f32x4_t*>(red + ((t++) * 64 + lane) * 4) = dw_hid[h][i][j];
#pragma unroll
      for (int i = 0; i < MT_H; ++i) *reinterpret_cast<f32x4_t*>(red + ((t++) * 64 + lane) * 4) = db_acc_in[i];
#pragma unroll
      for (int h = 0; h < (REG_HIDDEN > 0 ? REG_HIDDEN : 1); ++h)
#pragma unroll
        for (int i = 0; i < MT_H; ++i) *reinterpret_cast<f32x4_t*>(red + ((t++) * 64 + lane) * 4) = db_acc_hid[h][i];
    }
    __syncthreads();
    if (wave == 0) {
      int t = 0;
#pragma unroll
      for (int i = 0; i < MT_H; ++i)
#pragma unroll
        for (int j = 0; j < MT_I; ++j) dw_in[i][j] += *reinterpret_cast<const f32x4_t*>(red + ((t++) * 64 + lane) * 4);
#pragma unroll
      for (int i = 0; i < MT_O; ++i)
#pragma unroll
        for (int j = 0; j < MT_H; ++j) dw_out[i][j] += *reinterpret_cast<const f32x4_t*>(red + ((t++) * 64 + lane) * 4);
#pragma unroll
      for (int h = 0; h < (REG_HIDDEN > 0 ? REG_HIDDEN : 1); ++h)
#pragma unroll
        for (int i = 0; i < MT_H; ++i)
#pragma unroll
          for (int j = 0; j < MT_H; ++j) dw_hid[h][i][j] += *reinterpret_cast<const f32x4_t*>(red + ((t++) * 64 + lane) * 4);
#pragma unroll
      for (int i = 0; i < MT_H; ++i) db_acc_in[i] += *reinterpret_cast<const f32x4_t*>(red + ((t++) * 64 + lane) * 4);
#pragma unroll
      for (int h = 0; h < (REG_HIDDEN > 0 ? REG_HIDDEN : 1); ++h)
#pragma unroll
        for (int i = 0; i < MT_H; ++i) db_acc_hid[h][i] += *reinterpret_cast<const f32x4_t*>(red + ((t++) * 64 + lane) * 4);
    }
    __syncthreads();
  }
  if (wave != 0) return;

#pragma unroll
  for (int i = 0; i < MT_H; ++i)
#pragma unroll
    for (int j = 0; j < MT_I; ++j) flush_dw_tile(a.dw_in, a.d_hidden, a.d_in, i, j, lane, dw_in[i][j]);
#pragma unroll
  for (int i = 0; i < MT_O; ++i)
#pragma unroll
    for (int j = 0; j < MT_H; ++j) flush_dw_tile(a.dw_out, a.d_out, a.d_hidden, i, j, lane, dw_out[i][j]);
  if (regs_hold_hidden) {
#pragma unroll
    for (int h = 0; h < REG_HIDDEN; ++h)
      if (h < n_hid) {
        float* dst = a.dw_hid + (size_t)h * a.d_hidden * a.d_hidden;
#pragma unroll
        for (int i = 0; i < MT_H; ++i)
#pragma unroll
          for (int j = 0; j < MT_H; ++j) flush_dw_tile(dst, a.d_hidden, a.d_hidden, i, j, lane, dw_hid[h][i][j]);
      }
  }
  if (want_db) {
    // hidden / input biases: lane (n,g) reg r holds the partial sum of feature 16*mt + 4*g + r over its rows n
    auto fold_store = [&](f32x4_t s, int mt, float* dst, int width) {
      if (dst == nullptr) return;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float t = s[r];
        t += __shfl_xor(t, 1);
        t += __shfl_xor(t, 2);
        t += __shfl_xor(t, 4);
        t += __shfl_xor(t, 8);
        const int f = 16 * mt + 4 * (lane >> 4) + r;
        if ((lane & 15) == 0 && f < width) unsafeAtomicAdd(dst + f, t);
      }
    };
#pragma unroll
    for (int mt = 0; mt < MT_H; ++mt) fold_store(db_acc_in[mt], mt, a.db_in, a.d_hidden);
    if (regs_hold_hidden) {
#pragma unroll
      for (int h = 0; h < REG_HIDDEN; ++h)
        if (h < n_hid && a.db_hid != nullptr) {
#pragma unroll
          for (int mt = 0; mt < MT_H; ++mt) fold_store(db_acc_hid[h][mt], mt, a.db_hid + (size_t)h * a.d_hidden, a.d_hidden);
        }
    }
  }
}

// db_out = column sums of dy; tiny and memory-bound, done apart from the fused kernel.  The 256 threads of a workgroup
// cover 256 / cols rows at a time, cols = d_out rounded up to a power of two (a one-column dy keeps every lane busy).
template <typename T>
__global__ __launch_bounds__(256) void db_out_k(const uint16_t* dy, int64_t stride, int64_t rows, int d_out, int cols_log2, float* db_out) {
  __shared__ float part[256];
  const int cols = 1 << cols_log2, rows_per_turn = 256 >> cols_log2;
  const int c = threadIdx.x & (cols - 1), rl = threadIdx.x >> cols_log2;
  float s = 0.0f;
  if (c < d_out)
    for (int64_t r = (int64_t)blockIdx.x * rows_per_turn + rl; r < rows; r += (int64_t)gridDim.x * rows_per_turn)
      s += T::to_f32(dy[r * stride + c]);
  part[threadIdx.x] = s;
  __syncthreads();
  for (int h = 128; h >= cols; h >>= 1) {  // thread t and t + h hold the same column
    if ((int)threadIdx.x < h) part[threadIdx.x] += part[threadIdx.x + h];
    __syncthreads();
  }
  if ((int)threadIdx.x < d_out) unsafeAtomicAdd(db_out + threadIdx.x, part[threadIdx.x]);
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------
static int pad_to(int v, int m) { return (v + m - 1) / m * m; }

static int validate(int64_t rows, int d_in, int d_hidden, int d_out, int depth, int act, int dtype) {
  NF_REQUIRE(rows >= 0, NF_EINVAL, "rows negative");
  NF_REQUIRE(d_in >= 1 && d_in <= 64, NF_EINVAL, "d_in=%d outside 1..64", d_in);
  NF_REQUIRE(d_out >= 1 && d_out <= 64, NF_EINVAL, "d_out=%d outside 1..64", d_out);
  NF_REQUIRE(d_hidden >= 16 && d_hidden <= 64 && (d_hidden & (d_hidden - 1)) == 0, NF_EINVAL,
             "d_hidden=%d must be 16, 32 or 64", d_hidden);
  NF_REQUIRE(depth >= 1, NF_EINVAL, "depth=%d must be >= 1", depth);
  NF_REQUIRE(act >= NF_ACT_NONE && act <= NF_ACT_GELU, NF_EINVAL, "unknown activation %d", act);
  NF_REQUIRE(dtype_ok(dtype), NF_EINVAL, "unknown dtype code %d", dtype);
  return 0;
}

template <typename T, int KIN, int HP, int OUTP>
static int launch_fwd(const MlpArgs& a0, hipStream_t s) {
  MlpArgs a = a0;
  const int n_hid = a.depth - 1;
  const size_t lds = ((size_t)(HP / 16) * (KIN / 32) + (size_t)n_hid * (HP / 16) * (HP / 32) + (size_t)(OUTP / 16) * (HP / 32)) * 1024 +
                     ((size_t)HP + (size_t)n_hid * HP + OUTP) * 4;
  NF_REQUIRE(lds <= LDS_LIMIT, NF_EUNSUPPORTED, "weights of depth %d need %zu B of LDS (limit %zu)", a.depth, lds, LDS_LIMIT);
  // weights beyond half of LDS leave room for one workgroup per CU: give it eight waves to keep two per SIMD
  a.waves = lds > 76 * 1024 ? 8 : 4;
  const int64_t chunks = (a.rows + 31) / 32;
  int64_t blocks = (chunks + a.waves - 1) / a.waves;
  const int64_t cap = (int64_t)device_cus() * (lds > 76 * 1024 ? 1 : (lds > 40 * 1024 ? 2 : 3));
  if (blocks > cap) blocks = cap;
  constexpr int XC_OTHER = T::code == NF_BF16 ? 1 : 2;
  const void* kern = a.x_conv == 0 ? (const void*)mlp_fwd_k<T, KIN, HP, OUTP, 0> : (const void*)mlp_fwd_k<T, KIN, HP, OUTP, XC_OTHER>;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  void* args[] = {(void*)&a};
  const hipError_t le = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(64 * a.waves), args, lds, s);
  if (le != hipSuccess) return fail((int)le, "hipLaunchKernel(mlp_fwd): %s", hipGetErrorString(le));
  return check_launch("mlp_fwd");
}

template <typename T, int KIN, int HP, int OUTP, int REG_HIDDEN>
static int launch_bwd(const MlpArgs& a0, hipStream_t s) {
  MlpArgs a = a0;
  constexpr int KC_O = (OUTP + 31) / 32;
  constexpr int DZ_FEATS = HP > 32 * KC_O ? HP : 32 * KC_O;
  const int n_hid = a.depth - 1;
  const size_t w_bytes = ((size_t)(HP / 16) * (KIN / 32) + (size_t)(KIN / 16) * (HP / 32) + 2 * (size_t)n_hid * (HP / 16) * (HP / 32) +
                          (size_t)(HP / 16) * KC_O) * 1024 + ((size_t)HP + (size_t)n_hid * HP) * 4;
  const size_t per_wave = ((size_t)(KIN + (size_t)a.depth * HP + DZ_FEATS) * TPITCH + (size_t)a.depth * (HP / 16) * 2 * 2 * 64 * 2) * 2;
  // staging area for the cross-wave reduction (one wave's accumulators)
  const size_t red_bytes = ((size_t)(HP / 16) * (KIN / 16) + (size_t)(OUTP / 16) * (HP / 16) +
                            (size_t)(REG_HIDDEN > 0 ? REG_HIDDEN : 1) * (HP / 16) * (HP / 16) + (HP / 16) + (OUTP / 16) +
                            (size_t)(REG_HIDDEN > 0 ? REG_HIDDEN : 1) * (HP / 16)) * 64 * 16;
  int waves = 4;
  while (waves > 1 && w_bytes + waves * per_wave > LDS_LIMIT) waves >>= 1;
  size_t lds = w_bytes + waves * per_wave;
  if (waves > 1 && lds < w_bytes + red_bytes) lds = w_bytes + red_bytes;
  NF_REQUIRE(lds <= LDS_LIMIT, NF_EUNSUPPORTED, "backward of depth %d needs %zu B of LDS (limit %zu)", a.depth, lds, LDS_LIMIT);
  a.waves = waves;
  const int64_t chunks = (a.rows + 31) / 32;
  int64_t blocks = (chunks + waves - 1) / waves;
  const int64_t cap = (int64_t)device_cus() * (lds > 80 * 1024 ? 1 : 2);
  if (blocks > cap) blocks = cap;
  auto kern = mlp_bwd_k<T, KIN, HP, OUTP, REG_HIDDEN>;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(64 * waves), lds, s, a);
  if (int rc = check_launch("mlp_bwd")) return rc;
  if (a.db_out != nullptr) {
    int64_t b = (a.rows + 1023) / 1024;
    if (b > 1024) b = 1024;
    int cols_log2 = 0;
    while ((1 << cols_log2) < a.d_out) ++cols_log2;
    hipLaunchKernelGGL((db_out_k<T>), dim3((unsigned)b), dim3(256), 0, s, a.dy, a.dy_stride, a.rows, a.d_out, cols_log2, a.db_out);
    return check_launch("db_out");
  }
  return 0;
}

template <typename T>
static int dispatch_fwd(const MlpArgs& a, hipStream_t s) {
  const int kin = pad_to(a.d_in, 32), hp = a.d_hidden <= 32 ? 32 : 64, outp = a.d_out <= 16 ? 16 : 64;
  if (kin == 32 && hp == 64 && outp == 16) return launch_fwd<T, 32, 64, 16>(a, s);
  if (kin == 32 && hp == 64) return launch_fwd<T, 32, 64, 64>(a, s);
  if (kin == 64 && hp == 64 && outp == 16) return launch_fwd<T, 64, 64, 16>(a, s);
  if (kin == 64 && hp == 64) return launch_fwd<T, 64, 64, 64>(a, s);
  if (kin == 32 && outp == 16) return launch_fwd<T, 32, 32, 16>(a, s);
  if (kin == 32) return launch_fwd<T, 32, 32, 64>(a, s);
  if (outp == 16) return launch_fwd<T, 64, 32, 16>(a, s);
  return launch_fwd<T, 64, 32, 64>(a, s);
}

template <typename T, int REG_HIDDEN>
static int dispatch_bwd2(const MlpArgs& a, hipStream_t s) {
  const int kin = pad_to(a.d_in, 32), hp = a.d_hidden <= 32 ? 32 : 64, outp = a.d_out <= 16 ? 16 : 64;
  if (kin == 32 && hp == 64 && outp == 16) return launch_bwd<T, 32, 64, 16, REG_HIDDEN>(a, s);
  if (kin == 32 && hp == 64) return launch_bwd<T, 32, 64, 64, REG_HIDDEN>(a, s);
  if (kin == 64 && hp == 64 && outp == 16) return launch_bwd<T, 64, 64, 16, REG_HIDDEN>(a, s);
  if (kin == 64 && hp == 64) return launch_bwd<T, 64, 64, 64, REG_HIDDEN>(a, s);
  if (kin == 32 && outp == 16) return launch_bwd<T, 32, 32, 16, REG_HIDDEN>(a, s);
  if (kin == 32) return launch_bwd<T, 32, 32, 64, REG_HIDDEN>(a, s);
  if (outp == 16) return launch_bwd<T, 64, 32, 16, REG_HIDDEN>(a, s);
  return launch_bwd<T, 64, 32, 64, REG_HIDDEN>(a, s);
}

template <typename T>
static int dispatch_bwd(const MlpArgs& a, hipStream_t s) {
  // one hidden layer's dW fits in registers next to dW_in / dW_out; deeper nets use the memory path
  return a.depth - 1 <= 1 ? dispatch_bwd2<T, 1>(a, s) : dispatch_bwd2<T, 0>(a, s);
}

// ---------------------------------------------------------------------------------------
// Networks deeper than one launch covers
// ---------------------------------------------------------------------------------------
// A launch keeps every weight of its layers in LDS and (backward) every activation of a chunk on chip, which bounds
// the layers it can take.  Deeper networks run as a chain of launches over consecutive linear layers l0 .. l1-1
// (0 = input layer, depth = output layer).  The value handed from one launch to the next is the PRE-activation of layer
// l1-1, rounded to 16 bit: the launch behind applies the activation as it loads its rows (MlpArgs::in_act) and, in
// the backward, multiplies its dx by act'(x), so every launch is an ordinary "input layer, hidden layers, linear
// output layer" network and no elementwise pass runs in between.  The backward first replays the forward up to the
// last boundary, keeping each boundary's rows (rows * d_hidden * 2 bytes), then walks the launches last to first.

static int fwd_one(const MlpArgs& a, int dtype, hipStream_t s) {
  bool handled = false;
  const int rc = launch_mlp_fwd2(a, dtype, s, &handled);
  if (rc != 0 || handled) return rc;
  return dtype == NF_BF16 ? dispatch_fwd<BF16>(a, s) : dispatch_fwd<F16>(a, s);
}

static int bwd_one(const MlpArgs& a, int dtype, hipStream_t s) {
  bool handled = false;
  const int rc = launch_mlp_bwd2(a, dtype, s, &handled);
  if (rc != 0 || handled) return rc;
  NF_REQUIRE(a.x_conv == 0, NF_EUNSUPPORTED, "x_dtype != dtype needs depth == 2 and d_hidden > 32 in the backward");
  return dtype == NF_BF16 ? dispatch_bwd<BF16>(a, s) : dispatch_bwd<F16>(a, s);
}

// Most linear layers one forward launch holds in LDS (input and output layers priced at their widest).
static int fwd_max_linear(int d_hidden) {
  const int hp = d_hidden <= 32 ? 32 : 64;
  auto fits = [&](int n_linear) {
    const int n_hid = n_linear - 2;
    const size_t lds = ((size_t)(hp / 16) * 2 + (size_t)n_hid * (hp / 16) * (hp / 32) + (size_t)4 * (hp / 32)) * 1024 +
                       ((size_t)hp + (size_t)n_hid * hp + 64) * 4;
    return lds <= LDS_LIMIT;
  };
  int m = 2;
  while (fits(m + 1)) ++m;
  return m;
}

// Most linear layers one backward launch takes at full speed: the register-resident kernels of the 64-wide nets
// reach five (ReLU) or three; at width 16 / 32 the general kernel keeps one hidden layer's dW in registers, and its
// variant for more (partial dW through memory) costs several times a chain of those.
static int bwd_max_linear(int d_hidden, int act) {
  if (d_hidden > 32) return act == NF_ACT_RELU ? 5 : 3;
  return 3;
}

// Boundaries of the launches: n_linear layers in ceil(n_linear / max_per_launch) runs of near-equal length (each >= 2).
static std::vector<int> plan_launches(int n_linear, int max_per_launch) {
  const int n = (n_linear + max_per_launch - 1) / max_per_launch;
  std::vector<int> first(n + 1, 0);
  for (int k = 0; k <= n; ++k) first[k] = (int)((int64_t)n_linear * k / n);
  return first;
}

static size_t boundary_bytes(int64_t rows, int d_hidden) { return ((size_t)rows * d_hidden * 2 + 255) / 256 * 256; }

// Arguments of the launch over linear layers l0 .. l1-1 of network `a` (x / y / dy / dx are left to the caller).
static MlpArgs launch_args(const MlpArgs& a, int l0, int l1) {
  MlpArgs g = a;
  const int H = a.d_hidden, last = a.depth;
  const size_t hh = (size_t)H * H;
  auto W = [&](int l) { return l == 0 ? a.w_in : l == last ? a.w_out : a.w_hid + (size_t)(l - 1) * hh; };
  auto B = [&](int l) -> const uint16_t* {
    return l == 0 ? a.b_in : l == last ? a.b_out : (a.b_hid ? a.b_hid + (size_t)(l - 1) * H : nullptr);
  };
  auto DW = [&](int l) -> float* {
    if (a.dw_in == nullptr) return nullptr;  // forward
    return l == 0 ? a.dw_in : l == last ? a.dw_out : a.dw_hid + (size_t)(l - 1) * hh;
  };
  auto DB = [&](int l) -> float* {
    return l == 0 ? a.db_in : l == last ? a.db_out : (a.db_hid ? a.db_hid + (size_t)(l - 1) * H : nullptr);
  };
  const bool has_hid = l1 - l0 > 2;
  g.w_in = W(l0); g.b_in = B(l0); g.dw_in = DW(l0); g.db_in = DB(l0);
  g.w_out = W(l1 - 1); g.b_out = B(l1 - 1); g.dw_out = DW(l1 - 1); g.db_out = DB(l1 - 1);
  g.w_hid = has_hid ? W(l0 + 1) : nullptr; g.b_hid = has_hid ? B(l0 + 1) : nullptr;
  g.dw_hid = has_hid ? DW(l0 + 1) : nullptr; g.db_hid = has_hid ? DB(l0 + 1) : nullptr;
  g.d_in = l0 == 0 ? a.d_in : H;
  g.d_out = l1 - 1 == last ? a.d_out : H;
  g.depth = l1 - l0 - 1;
  g.in_act = l0 == 0 ? NF_ACT_NONE : a.act;
  g.x_conv = l0 == 0 ? a.x_conv : 0;
  return g;
}

static void set_rows(MlpArgs& g, const uint16_t* x, int64_t x_stride, uint16_t* y, int64_t y_stride, const uint16_t* dy,
                     int64_t dy_stride, uint16_t* dx, int64_t dx_stride) {
  g.x = x; g.x_stride = x_stride; g.y = y; g.y_stride = y_stride;
  g.dy = dy; g.dy_stride = dy_stride; g.dx = dx; g.dx_stride = dx_stride;
  g.x_vec = vec_load_ok(x, x_stride, g.d_in);
  g.y_vec = y ? vec_store_ok(y, y_stride, g.d_out) : 0;
  g.dy_vec = dy ? vec_load_ok(dy, dy_stride, g.d_out) : 0;
  g.dx_vec = dx ? vec_store_ok(dx, dx_stride, g.d_in) : 0;
}

// ---------------------------------------------------------------------------------------
// One hidden layer (depth 1, d_in -> 64 -> d_out, ReLU) on the backward kernels built for two.
// Behind a ReLU every hidden value is >= 0, so an identity layer with a ReLU of its own between the hidden layer and the
// output changes nothing: h2 = relu(I h1) = h1 bit for bit (one non-zero term per float32 sum, a value that is already
// a 16-bit number), the gradient crosses the identity unchanged, meets the same gate and rounds to the 16-bit number it
// already is.  The extra 64 x 64 products cost a third of the two-layer kernel's work, which is still several times
// quicker than the general kernel; the identity's own weight gradient goes to a sink nobody reads.
// The identity (one per 16-bit type) and the sink are file-scope device arrays; the identity is written by a tiny kernel on
// the caller's stream in front of every such backward (no cross-stream ordering to rely on, same values every time), and
// concurrent calls share the sink, whose contents mean nothing.
// ---------------------------------------------------------------------------------------
static __device__ __align__(256) uint16_t identity_hidden[2][64 * 64];  // [bfloat16, float16]
static __device__ __align__(256) float identity_sink[64 * 64 + 64];     // dW (float32, or 16-bit rounded) and db of the identity

__global__ __launch_bounds__(256) void identity_fill_k(uint16_t* w) {
  const int i = blockIdx.x * 256 + threadIdx.x;  // 2 x 4096 elements
  const int e = i & 4095;
  w[i] = (e >> 6) == (e & 63) ? (i < 4096 ? (uint16_t)0x3F80u : (uint16_t)0x3C00u) : (uint16_t)0u;
}

static bool identity_layer_applies(int d_hidden, int depth, int act, int dtype) {
  return depth == 1 && d_hidden == 64 && act == NF_ACT_RELU && (dtype == NF_BF16 || dtype == NF_F16);
}

// the identity in `dtype` and the sink, on the current device; the fill is queued on `s`
static int identity_layer(int dtype, hipStream_t s, const uint16_t** w, float** sink) {
  uint16_t* base = nullptr;
  float* sk = nullptr;
  hipError_t e = hipGetSymbolAddress((void**)&base, HIP_SYMBOL(identity_hidden));
  if (e == hipSuccess) e = hipGetSymbolAddress((void**)&sk, HIP_SYMBOL(identity_sink));
  if (e != hipSuccess) return fail((int)e, "hipGetSymbolAddress(identity layer): %s", hipGetErrorString(e));
  hipLaunchKernelGGL(identity_fill_k, dim3(2 * 4096 / 256), dim3(256), 0, s, base);
  if (int rc = check_launch("identity_fill")) return rc;
  *w = base + (dtype == NF_BF16 ? 0 : 4096);
  *sink = sk;
  return 0;
}

}  // namespace nf

using namespace nf;

extern "C" int64_t nf_mlp_workspace_bytes(int64_t rows, int d_hidden, int depth, int act, int backward, int dtype) {
  if (rows <= 0 || depth < 1 || d_hidden < 1) return 0;
  if (dtype == NF_F32) return backward ? (int64_t)mlp32_bwd_workspace_bytes(rows, d_hidden, depth) : 0;
  const int n_linear = depth + 1;
  const int n = (int)plan_launches(n_linear, backward ? bwd_max_linear(d_hidden, act) : fwd_max_linear(d_hidden)).size() - 1;
  if (n <= 1) return 0;
  // forward: two boundaries alive at a time; backward: every boundary plus two gradient buffers
  return (int64_t)boundary_bytes(rows, d_hidden) * (backward ? (n - 1) + 2 : 2);
}

extern "C" int nf_mlp_fwd(const void* x, int64_t x_stride, void* y, int64_t y_stride, const void* w_in, const void* b_in,
                          const void* w_hid, const void* b_hid, const void* w_out, const void* b_out, int64_t rows,
                          int d_in, int d_hidden, int d_out, int depth, int act, int dtype, int x_dtype, void* workspace,
                          int64_t workspace_bytes, void* stream) {
  if (int rc = validate(rows, d_in, d_hidden, d_out, depth, act, dtype)) return rc;
  NF_REQUIRE(dtype == NF_F32 ? x_dtype == NF_F32 : (x_dtype == NF_F16 || x_dtype == NF_BF16), NF_EUNSUPPORTED,
             "x_dtype code %d with dtype code %d: float32 with float32, float16 or bfloat16 with the 16-bit types", x_dtype, dtype);
  if (rows == 0) return 0;
  NF_REQUIRE(x && y && w_in && w_out, NF_EINVAL, "NULL pointer argument");
  NF_REQUIRE(depth == 1 || w_hid, NF_EINVAL, "w_hid is NULL but depth=%d", depth);
  NF_REQUIRE(x_stride >= d_in && y_stride >= d_out, NF_EINVAL, "row stride smaller than row width");
  if (dtype == NF_F32)
    return mlp32_fwd((const float*)x, x_stride, (float*)y, y_stride, (const float*)w_in, (const float*)b_in, (const float*)w_hid,
                     (const float*)b_hid, (const float*)w_out, (const float*)b_out, rows, d_in, d_hidden, d_out, depth, act,
                     (hipStream_t)stream);
  MlpArgs a = {};
  a.w_in = (const uint16_t*)w_in; a.b_in = (const uint16_t*)b_in; a.w_hid = (const uint16_t*)w_hid;
  a.b_hid = (const uint16_t*)b_hid; a.w_out = (const uint16_t*)w_out; a.b_out = (const uint16_t*)b_out;
  a.rows = rows; a.d_in = d_in; a.d_hidden = d_hidden; a.d_out = d_out; a.depth = depth; a.act = act;
  a.in_act = NF_ACT_NONE;
  a.x_conv = x_dtype == dtype ? 0 : (x_dtype == NF_F16 ? 1 : 2);
  set_rows(a, (const uint16_t*)x, x_stride, (uint16_t*)y, y_stride, nullptr, 0, nullptr, 0);
  hipStream_t s = (hipStream_t)stream;
  const std::vector<int> first = plan_launches(depth + 1, fwd_max_linear(d_hidden));
  const int n = (int)first.size() - 1;
  if (n == 1) return fwd_one(a, dtype, s);
  const size_t buf = boundary_bytes(rows, d_hidden);
  NF_REQUIRE(workspace != nullptr && workspace_bytes >= (int64_t)(2 * buf), NF_EINVAL,
             "forward of depth %d runs as %d launches and needs a workspace of %zu bytes (nf_mlp_workspace_bytes)", depth, n,
             2 * buf);
  NF_REQUIRE((uintptr_t)workspace % 16 == 0, NF_EINVAL, "workspace must be 16-byte aligned");
  uint16_t* bound[2] = {(uint16_t*)workspace, (uint16_t*)((char*)workspace + buf)};
  for (int k = 0; k < n; ++k) {
    MlpArgs g = launch_args(a, first[k], first[k + 1]);
    set_rows(g, k == 0 ? a.x : bound[(k - 1) & 1], k == 0 ? a.x_stride : d_hidden, k == n - 1 ? a.y : bound[k & 1],
             k == n - 1 ? a.y_stride : d_hidden, nullptr, 0, nullptr, 0);
    if (int rc = fwd_one(g, dtype, s)) return rc;
  }
  return 0;
}

extern "C" int nf_mlp_bwd(const void* x, int64_t x_stride, const void* dy, int64_t dy_stride, void* dx, int64_t dx_stride,
                          const void* w_in, const void* b_in, const void* w_hid, const void* b_hid, const void* w_out,
                          const void* b_out, float* dw_in, float* db_in, float* dw_hid, float* db_hid, float* dw_out,
                          float* db_out, int64_t rows, int d_in, int d_hidden, int d_out, int depth, int act, int dtype,
                          int x_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = validate(rows, d_in, d_hidden, d_out, depth, act, dtype)) return rc;
  NF_REQUIRE(dtype == NF_F32 ? x_dtype == NF_F32 : (x_dtype == NF_F16 || x_dtype == NF_BF16), NF_EUNSUPPORTED,
             "x_dtype code %d with dtype code %d: float32 with float32, float16 or bfloat16 with the 16-bit types", x_dtype, dtype);
  if (rows == 0) return 0;
  NF_REQUIRE(x && dy && w_in && w_out && dw_in && dw_out, NF_EINVAL, "NULL pointer argument");
  NF_REQUIRE(depth == 1 || (w_hid && dw_hid), NF_EINVAL, "w_hid / dw_hid is NULL but depth=%d", depth);
  NF_REQUIRE(x_stride >= d_in && dy_stride >= d_out && (dx == nullptr || dx_stride >= d_in), NF_EINVAL,
             "row stride smaller than row width");
  if (dtype == NF_F32)
    return mlp32_bwd((const float*)x, x_stride, (const float*)dy, dy_stride, (float*)dx, dx_stride, (const float*)w_in,
                     (const float*)b_in, (const float*)w_hid, (const float*)b_hid, (const float*)w_out, dw_in, db_in, dw_hid,
                     db_hid, dw_out, db_out, rows, d_in, d_hidden, d_out, depth, act, workspace, workspace_bytes,
                     (hipStream_t)stream);
  MlpArgs a = {};
  a.w_in = (const uint16_t*)w_in; a.b_in = (const uint16_t*)b_in; a.w_hid = (const uint16_t*)w_hid;
  a.b_hid = (const uint16_t*)b_hid; a.w_out = (const uint16_t*)w_out; a.b_out = (const uint16_t*)b_out;
  a.dw_in = dw_in; a.db_in = db_in; a.dw_hid = dw_hid; a.db_hid = db_hid; a.dw_out = dw_out; a.db_out = db_out;
  a.rows = rows; a.d_in = d_in; a.d_hidden = d_hidden; a.d_out = d_out; a.depth = depth; a.act = act;
  a.in_act = NF_ACT_NONE;
  a.x_conv = x_dtype == dtype ? 0 : (x_dtype == NF_F16 ? 1 : 2);
  set_rows(a, (const uint16_t*)x, x_stride, nullptr, 0, (const uint16_t*)dy, dy_stride, (uint16_t*)dx, dx_stride);
  hipStream_t s = (hipStream_t)stream;
  if (identity_layer_applies(d_hidden, depth, act, dtype)) {
    float* sink = nullptr;
    if (int rc = identity_layer(dtype, s, &a.w_hid, &sink)) return rc;
    a.b_hid = nullptr; a.dw_hid = sink; a.db_hid = nullptr; a.depth = 2;
    return bwd_one(a, dtype, s);
  }
  const std::vector<int> first = plan_launches(depth + 1, bwd_max_linear(d_hidden, act));
  const int n = (int)first.size() - 1;
  if (n == 1) return bwd_one(a, dtype, s);
  const size_t buf = boundary_bytes(rows, d_hidden);
  const size_t need = buf * (size_t)(n - 1 + 2);
  if (workspace == nullptr || workspace_bytes < (int64_t)need) {
    // no scratch: the one-launch general kernel (partial dW through memory) where the network fits it
    const int rc = bwd_one(a, dtype, s);
    if (rc != NF_EUNSUPPORTED) return rc;
    return fail(NF_EINVAL, "backward of depth %d runs as %d launches and needs a workspace of %zu bytes (nf_mlp_workspace_bytes)",
                depth, n, need);
  }
  NF_REQUIRE((uintptr_t)workspace % 16 == 0, NF_EINVAL, "workspace must be 16-byte aligned");
  if (a.x_conv != 0) {
    // Only the first launch sees x, and it runs last: by then the launches behind it have added into the caller's
    // accumulators.  Whatever would make it refuse the conversion is therefore checked before anything is launched,
    // so that a caller who casts x and calls again does not count the later layers' gradients twice.
    const MlpArgs g0 = launch_args(a, first[0], first[1]);
    const bool aligned = ((uintptr_t)x % 8 == 0) && (x_stride % 4 == 0) && (d_in % 4 == 0) &&
                         (dx == nullptr || ((uintptr_t)dx % 8 == 0 && dx_stride % 4 == 0));
    NF_REQUIRE(g0.depth == 2 && d_hidden > 32 && act == NF_ACT_RELU && aligned, NF_EUNSUPPORTED,
               "x_dtype != dtype: the backward converts x on the fly only in a first launch of three linear layers, d_hidden > 32, "
               "ReLU and 8-byte aligned rows (nothing was launched; cast x and call again)");
  }
  auto bound = [&](int k) { return (uint16_t*)((char*)workspace + (size_t)k * buf); };       // output of launch k, k < n-1
  auto grad = [&](int k) { return (uint16_t*)((char*)workspace + (size_t)(n - 1 + (k & 1)) * buf); };  // d/d(input of launch k)
  // replay the forward up to the last boundary
  for (int k = 0; k + 1 < n; ++k) {
    MlpArgs g = launch_args(a, first[k], first[k + 1]);
    g.dw_in = g.dw_hid = g.dw_out = nullptr;
    set_rows(g, k == 0 ? a.x : bound(k - 1), k == 0 ? a.x_stride : d_hidden, bound(k), d_hidden, nullptr, 0, nullptr, 0);
    if (int rc = fwd_one(g, dtype, s)) return rc;
  }
  for (int k = n - 1; k >= 0; --k) {
    MlpArgs g = launch_args(a, first[k], first[k + 1]);
    set_rows(g, k == 0 ? a.x : bound(k - 1), k == 0 ? a.x_stride : d_hidden, nullptr, 0, k == n - 1 ? a.dy : grad(k + 1),
             k == n - 1 ? a.dy_stride : d_hidden, k == 0 ? a.dx : grad(k), k == 0 ? a.dx_stride : d_hidden);
    if (int rc = bwd_one(g, dtype, s)) return rc;
  }
  return 0;
}


extern "C" int64_t nf_mlp_bwd_rounded_workspace_bytes(int d_in, int d_hidden, int d_out) {
  if (d_in < 1 || d_hidden < 1 || d_out < 1) return 0;
  return (int64_t)mlp_bwd2_w8_rounded_bytes(d_in, d_hidden, d_out);
}

extern "C" int nf_mlp_bwd_rounded(const void* x, int64_t x_stride, const void* dy, int64_t dy_stride, void* dx, int64_t dx_stride,
                                  const void* w_in, const void* b_in, const void* w_hid, const void* b_hid, const void* w_out,
                                  const void* b_out, void* dw_in, void* db_in, void* dw_hid, void* db_hid, void* dw_out,
                                  void* db_out, int64_t rows, int d_in, int d_hidden, int d_out, int depth, int act, int dtype,
                                  int x_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = validate(rows, d_in, d_hidden, d_out, depth, act, dtype)) return rc;
  NF_REQUIRE(dtype != NF_F32 && (x_dtype == NF_F16 || x_dtype == NF_BF16), NF_EUNSUPPORTED,
             "rounded weight gradients: 16-bit tensors only (dtype code %d, x_dtype code %d)", dtype, x_dtype);
  NF_REQUIRE(rows > 0, NF_EUNSUPPORTED, "rounded weight gradients: no rows (the buffers would stay unwritten)");
  const bool identity = identity_layer_applies(d_hidden, depth, act, dtype);  // one hidden layer: see identity_layer()
  NF_REQUIRE(x && dy && w_in && w_out && dw_in && dw_out && (identity || (w_hid && dw_hid)), NF_EINVAL, "NULL pointer argument");
  NF_REQUIRE(x_stride >= d_in && dy_stride >= d_out && (dx == nullptr || dx_stride >= d_in), NF_EINVAL,
             "row stride smaller than row width");
  const int64_t need = nf_mlp_bwd_rounded_workspace_bytes(d_in, d_hidden, d_out);
  NF_REQUIRE(workspace != nullptr && workspace_bytes >= need && (uintptr_t)workspace % 16 == 0, NF_EINVAL,
             "rounded weight gradients need a 16-byte aligned workspace of %lld bytes (nf_mlp_bwd_rounded_workspace_bytes)",
             (long long)need);
  MlpArgs a = {};
  a.w_in = (const uint16_t*)w_in; a.b_in = (const uint16_t*)b_in; a.w_hid = (const uint16_t*)w_hid;
  a.b_hid = (const uint16_t*)b_hid; a.w_out = (const uint16_t*)w_out; a.b_out = (const uint16_t*)b_out;
  a.rows = rows; a.d_in = d_in; a.d_hidden = d_hidden; a.d_out = d_out; a.depth = depth; a.act = act;
  a.in_act = NF_ACT_NONE;
  a.x_conv = x_dtype == dtype ? 0 : (x_dtype == NF_F16 ? 1 : 2);
  set_rows(a, (const uint16_t*)x, x_stride, nullptr, 0, (const uint16_t*)dy, dy_stride, (uint16_t*)dx, dx_stride);
  if (identity) {
    float* sink = nullptr;
    if (int rc = identity_layer(dtype, (hipStream_t)stream, &a.w_hid, &sink)) return rc;
    a.b_hid = nullptr; a.depth = 2;
    dw_hid = nullptr; db_hid = nullptr;  // the sum over the slots leaves out pieces without a destination
  }
  void* const out[6] = {dw_in, db_in, dw_hid, db_hid, dw_out, db_out};
  bool handled = false;
  const int rc = launch_mlp_bwd2_w8_rounded(a, dtype, out, workspace, (hipStream_t)stream, &handled);
  if (rc != 0 || handled) return rc;
  return fail(NF_EUNSUPPORTED, "rounded weight gradients: built for one hidden-to-hidden layer, d_hidden = 64, d_in <= 64, d_out <= 64, "
                               "ReLU, 8-byte aligned rows and (beyond d_in 32 / d_out 16) x stored like the weights (nothing was launched; use nf_mlp_bwd)");
}
