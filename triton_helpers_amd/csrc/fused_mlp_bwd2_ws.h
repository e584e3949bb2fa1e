// One-hidden-layer ReLU backward (d_in <= 64, d_hidden = 64, d_out <= 64) with the work of a workgroup split by ROLE:
// sixteen waves, two "chain" waves and two "gradient" waves per SIMD.
//
// What the split is for.  A wave issues in order and its vector instructions do not start while one of its own matrix
// products is in flight (measured: a product followed by eight independent vector instructions takes 16 + 8 x 4
// clocks), so a SIMD's matrix core and vector ALU only overlap across waves; and the weight gradients of a 64-wide
// network (up to 48 tiles = 192 accumulator registers) leave no room for the rest of the backward in the same wave.
//
//   * a round covers four 32-row panels.  A chain wave owns 16 rows of a panel per round (two chain waves per panel, so
//     that a SIMD has a second chain to run while the first waits for weight fragments or a barrier): it recomputes the
//     forward, carries the gradient back through the three layers (all the packing / gating vector work) and writes dx.
//     It holds no weight-gradient accumulator.
//   * the two gradient waves of a panel hold its weight-gradient accumulators for the whole launch, half of the
//     output features each (at most 24 tiles = 96 of the 128 registers a wave has at four waves per SIMD; the B operands
//     of a section's products are therefore taken two at a time).  The chain waves park the operands of dW = dz^T h
//     (row-major, 16 bit) in the panel; the gradient waves read them back transposed (ds_read_b64_tr_b16) and run the
//     products of the panel while the chain waves are busy with vector work.
//   (With four chain waves of 32 rows each -- twelve waves, 168 registers -- the same kernel takes 12 - 15 % longer:
//   64 -> 64 -> 64 -> 64 with biases 160 against 139 us per 2^20 rows.  The template keeps both.)
//
// The roles meet at three workgroup barriers per round.  A panel has one area per section ({h2, dy},
// {h1, dz2}, {dz1, x}); a section is announced by the barrier in front of the NEXT section's stores, by which time its
// own stores have long landed, and it is overwritten a full round later, after the gradient wave has passed three more
// barriers.  Rows past the end of the batch read as zero through the buffer descriptors (a zero dy row contributes
// nothing to any gradient) and their dx stores are dropped, so every wave runs every round and reaches every barrier.
#pragma once

#include "fused_mlp_bwd2_kernels.h"

namespace nf {

// panels per round, gradient waves, chain waves (one or two per panel)
constexpr int WS_CHAIN = 4, WS_GRAD = 8, WS_CHAIN_WAVES = 8, WS_WAVES = WS_CHAIN_WAVES + WS_GRAD;
// dwords per panel row for 64 / 32 / 16 features: the features plus padding that spreads the rows over the banks
constexpr int ws_stride(int features) { return features == 64 ? 34 : features == 32 ? 20 : 12; }
constexpr int ws_panel(int features) { return 32 * ws_stride(features); }  // dwords per 32-row panel

// fragment of K-chunk kc (chain order) of row tile nt -> row-major panel with S dwords per row
template <int S, bool BOTH_HALVES>
__device__ __forceinline__ void ws_park(uint32_t* panel, const Frag& f, int nt, int kc, int lane) {
  uint32_t* p = panel + (16 * nt + (lane & 15)) * S + 16 * kc + 2 * (lane >> 4);
  *reinterpret_cast<uint2*>(p) = make_uint2(f.w[0], f.w[1]);
  if (BOTH_HALVES) *reinterpret_cast<uint2*>(p + 8) = make_uint2(f.w[2], f.w[3]);
}
// operand of a product over the panel's 32 rows: lane (i, g) <- feature 16 * tile + i of rows g + 4k and 16 + g + 4k
template <int S>
__device__ __forceinline__ Frag ws_operand(const uint32_t* panel, int tile, int lane) {
  const int i = lane & 15, g = lane >> 4;
  const uint32_t* p = panel + (g + 4 * (i >> 2)) * S + 8 * tile + 2 * (i & 3);
  typedef tr_v4i16 __attribute__((address_space(3))) * lds_ptr;
  const tr_v4i16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p);
  const tr_v4i16 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 16 * S));
  Frag f;
  const uint2 a = __builtin_bit_cast(uint2, lo), b = __builtin_bit_cast(uint2, hi);
  f.w[0] = a.x;
  f.w[1] = a.y;
  f.w[2] = b.x;
  f.w[3] = b.y;
  return f;
}

// Workgroup barrier that waits for this wave's LDS traffic only: global loads (the next chunk's rows) and the dx
// stores stay in flight across it.
__device__ __forceinline__ void ws_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int KIN, int OUTP>
struct WsShape {
  static constexpr int KC_IN = KIN / 32, KC_O = (OUTP + 31) / 32, MT_H = 4, MT_I = KIN / 16, MT_O = OUTP / 16;
  static constexpr int FRAGS = MT_H * KC_IN + MT_H * 2 + MT_I * 2 + MT_H * 2 + MT_H * KC_O;  // W_in, W_hid, W_in^T, W_hid^T, W_out^T
  static constexpr size_t W_BYTES = (size_t)FRAGS * 1024 + 2 * 64 * 4;
  static constexpr int AREA_A = ws_panel(64) + ws_panel(OUTP);  // {h2 | dy}
  static constexpr int AREA_B = 2 * ws_panel(64);               // {h1 | dz2}
  static constexpr int AREA_C = ws_panel(64) + ws_panel(KIN);   // {dz1 | x}
  static constexpr int WAVE_DWORDS = AREA_A + AREA_B + AREA_C;
  // a gradient wave of half h holds the rows 32 h .. 32 h + 31 of dW_in and dW_hid, and of dW_out when it is 64 rows
  // high (a 16-row dW_out belongs to half 0): tiles [dW_in 2 x MT_I | dW_hid 2 x 4 | dW_out RO x 4]
  static constexpr int RO = MT_O == 4 ? 2 : 1;
  static constexpr int T_IN = 0, T_HID = 2 * MT_I, T_OUT = T_HID + 2 * MT_H, TILES = T_OUT + RO * MT_H;
  static constexpr int NBIAS = 4 + RO;  // db_in (2), db_hid (2), db_out (RO)
  // the closing sum parks one half's tiles of the four chain waves' chunks in LDS at a time
  static constexpr size_t RED_BYTES = (size_t)WS_CHAIN * ((size_t)TILES * 1024 + (size_t)NBIAS * 256);
  static constexpr size_t RUN_BYTES = W_BYTES + (size_t)WS_CHAIN * WAVE_DWORDS * 4;
  static constexpr size_t LDS = RUN_BYTES > RED_BYTES ? RUN_BYTES : RED_BYTES;
  static_assert(LDS <= 160 * 1024, "LDS budget of the role-split backward");
};

// XC: how x / dx are stored (MlpArgs::x_conv, 0 or the other 16-bit type); B: the network has biases or bias
// gradients are wanted (false: accumulators start at zero and no row sums are kept).
template <typename T, int KIN, int OUTP, int XC, bool B, int CH = WS_CHAIN_WAVES>
__global__ __launch_bounds__(64 * (CH + WS_GRAD), 1) void mlp_bwd2_ws_k(MlpArgs a) {
  using SH = WsShape<KIN, OUTP>;
  // CH chain waves share the WS_CHAIN panels of a round: four own a 32-row panel each, eight a 16-row half each
  static_assert(CH == WS_CHAIN || CH == 2 * WS_CHAIN, "four or eight chain waves");
  constexpr int NT = CH == WS_CHAIN ? 2 : 1, WAVES = CH + WS_GRAD;
  // B operands of a section's products held at a time: all four with 168 registers per wave, two with 128
  constexpr int JB = CH == WS_CHAIN ? 4 : 2;
  constexpr int KC_IN = SH::KC_IN, KC_O = SH::KC_O, MT_H = SH::MT_H, MT_I = SH::MT_I, MT_O = SH::MT_O;
  constexpr int TILES = SH::TILES, NBIAS = SH::NBIAS;
  constexpr int S_H = ws_stride(64), S_X = ws_stride(KIN), S_Y = ws_stride(OUTP), P_H = ws_panel(64);
  constexpr int DY_HALVES = OUTP > 16 ? 2 : 1;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x;
  constexpr int nthreads = 64 * WAVES;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // a chain wave's panel and the first 16-row tile it owns there
  const int pd = CH == WS_CHAIN ? wave : wave >> 1, pt0 = CH == WS_CHAIN ? 0 : wave & 1;

  uint16_t* f_in = reinterpret_cast<uint16_t*>(smem);       // W_in    [MT_H][KC_IN]
  uint16_t* f_hid = f_in + MT_H * KC_IN * FRAG_ELEMS;       // W_hid   [MT_H][2]
  uint16_t* t_in = f_hid + MT_H * 2 * FRAG_ELEMS;           // W_in^T  [MT_I][2]
  uint16_t* t_hid = t_in + MT_I * 2 * FRAG_ELEMS;           // W_hid^T [MT_H][2]
  uint16_t* t_out = t_hid + MT_H * 2 * FRAG_ELEMS;          // W_out^T [MT_H][KC_O]
  float* bias_in = reinterpret_cast<float*>(t_out + MT_H * KC_O * FRAG_ELEMS);
  float* bias_hid = bias_in + 64;
  uint32_t* panels = reinterpret_cast<uint32_t*>(bias_hid + 64);  // [WS_CHAIN][A | B | C]

  const int64_t n_chunks = (a.rows + 31) / 32;
  const int64_t per_round = (int64_t)gridDim.x * WS_CHAIN;
  const int rounds = (int)((n_chunks + per_round - 1) / per_round);
  const bool chain = wave < CH;

  // the chain waves ask for their first rows before the weights are staged
  const __amdgpu_buffer_rsrc_t rs_x = rows_rsrc(a.x, a.rows, a.x_stride), rs_dy = rows_rsrc(a.dy, a.rows, a.dy_stride),
                               rs_dx = rows_rsrc(a.dx, a.dx != nullptr ? a.rows : 0, a.dx_stride);
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
  // a chunk past the end (a wave without work in the last round) reads zeros and stores nothing
  auto at = [&](int64_t chunk, int nt, int64_t stride, uint32_t off) {
    return chunk < n_chunks ? off + (uint32_t)((chunk * 32 + 16 * nt) * stride * 2) : OUT_OF_RANGE;
  };
  auto load_x = [&](int64_t chunk, int nt, int kc) {
    const buf_v2u lo = __builtin_amdgcn_raw_buffer_load_b64(rs_x, at(chunk, nt, a.x_stride, off_x[kc][0]), 0, 0);
    const buf_v2u hi = __builtin_amdgcn_raw_buffer_load_b64(rs_x, at(chunk, nt, a.x_stride, off_x[kc][1]), 0, 0);
    Frag f;
    f.w[0] = lo[0]; f.w[1] = lo[1]; f.w[2] = hi[0]; f.w[3] = hi[1];
    return f;
  };
  auto load_dy = [&](int64_t chunk, int nt, int kc) {
    const buf_v2u lo = __builtin_amdgcn_raw_buffer_load_b64(rs_dy, at(chunk, nt, a.dy_stride, off_dy[kc][0]), 0, 0);
    Frag f;
    f.w[0] = lo[0]; f.w[1] = lo[1]; f.w[2] = 0u; f.w[3] = 0u;
    if constexpr (DY_HALVES == 2) {
      const buf_v2u hi = __builtin_amdgcn_raw_buffer_load_b64(rs_dy, at(chunk, nt, a.dy_stride, off_dy[kc][DY_HALVES - 1]), 0, 0);
      f.w[2] = hi[0]; f.w[3] = hi[1];
    }
    return f;
  };
  const int64_t first_chunk = (int64_t)blockIdx.x * WS_CHAIN + pd;
  Frag nx[NT][KC_IN], ndy[NT][KC_O];
  if (chain) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int kc = 0; kc < KC_IN; ++kc) nx[nt][kc] = load_x(first_chunk, pt0 + nt, kc);
#pragma unroll
      for (int kc = 0; kc < KC_O; ++kc) ndy[nt][kc] = load_dy(first_chunk, pt0 + nt, kc);
    }
  }

  stage_weight_frags<true, false, nthreads>(f_in, a.w_in, a.d_hidden, a.d_in, MT_H, KC_IN, tid, nthreads);
  stage_weight_frags<true, false, nthreads>(f_hid, a.w_hid, a.d_hidden, a.d_hidden, MT_H, 2, tid, nthreads);
  stage_weight_frags<true, true, nthreads>(t_in, a.w_in, a.d_hidden, a.d_in, MT_I, 2, tid, nthreads);
  stage_weight_frags<true, true, nthreads>(t_hid, a.w_hid, a.d_hidden, a.d_hidden, MT_H, 2, tid, nthreads);
  stage_weight_frags<true, true, nthreads>(t_out, a.w_out, a.d_out, a.d_hidden, MT_H, KC_O, tid, nthreads);
  stage_bias<T>(bias_in, a.b_in, a.d_hidden, 64, tid, nthreads);
  stage_bias<T>(bias_hid, a.b_hid, a.d_hidden, 64, tid, nthreads);
  __syncthreads();

  // a gradient wave's accumulators: tile t of [dW_in (2 x MT_I) | dW_hid (2 x MT_H) | dW_out (RO x MT_H)] of its half
  // of the output features, row sums [db_in (2) | db_hid (2) | db_out (RO)]
  f32x4_t acc_dw[TILES];
  float acc_db[NBIAS];

  if (chain) {
    // ------------------------------------------------------------------ chain waves
    uint32_t* area_a = panels + (size_t)pd * SH::WAVE_DWORDS;
    uint32_t* area_b = area_a + SH::AREA_A;
    uint32_t* area_c = area_b + SH::AREA_B;
    for (int round = 0; round < rounds; ++round) {
      const int64_t chunk = first_chunk + (int64_t)round * per_round;
      Frag in[NT][2], h1[NT][2], h2[NT][2], dz[NT][2];
      f32x4_t acc[NT][4];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int kc = 0; kc < KC_IN; ++kc) {
          in[nt][kc] = XC == 0 ? nx[nt][kc] : convert_frag(nx[nt][kc], XC);
          nx[nt][kc] = load_x(chunk + per_round, pt0 + nt, kc);
        }
#pragma unroll
        for (int kc = 0; kc < KC_O; ++kc) {
          dz[nt][kc] = ndy[nt][kc];
          ndy[nt][kc] = load_dy(chunk + per_round, pt0 + nt, kc);
        }
      }
      // ---- forward recompute ----
      layer_nt<T, NT, MT_H, KC_IN, B ? 1 : 0>(acc, in, f_in, bias_in, lane);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT_H; ++mt) {
          h1[nt][mt >> 1].w[2 * (mt & 1)] = relu_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]));
          h1[nt][mt >> 1].w[2 * (mt & 1) + 1] = relu_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]));
        }
      layer_nt<T, NT, MT_H, 2, B ? 1 : 0>(acc, h1, f_hid, bias_hid, lane);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT_H; ++mt) {
          h2[nt][mt >> 1].w[2 * (mt & 1)] = relu_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]));
          h2[nt][mt >> 1].w[2 * (mt & 1) + 1] = relu_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]));
        }
      auto gates = [&](const Frag (&h)[NT][2]) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT_H; ++mt) {
            dz[nt][mt >> 1].w[2 * (mt & 1)] = relu_gate_pk(pack2<T>(acc[nt][mt][0], acc[nt][mt][1]), h[nt][mt >> 1].w[2 * (mt & 1)]);
            dz[nt][mt >> 1].w[2 * (mt & 1) + 1] = relu_gate_pk(pack2<T>(acc[nt][mt][2], acc[nt][mt][3]), h[nt][mt >> 1].w[2 * (mt & 1) + 1]);
          }
      };
      ws_barrier();  // announces {dz1, x} of the previous round
      // ---- section A: {h2, dy} ----
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int kc = 0; kc < 2; ++kc) ws_park<S_H, true>(area_a, h2[nt][kc], pt0 + nt, kc, lane);
#pragma unroll
        for (int kc = 0; kc < KC_O; ++kc) ws_park<S_Y, (OUTP > 16)>(area_a + P_H, dz[nt][kc], pt0 + nt, kc, lane);
      }
      layer_nt<T, NT, MT_H, KC_O, 0>(acc, dz, t_out, nullptr, lane);  // dh2 = W_out^T dy
      gates(h2);                                                      // dz2
      ws_barrier();  // announces {h2, dy}
      // ---- section B: {h1, dz2} ----
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int kc = 0; kc < 2; ++kc) {
          ws_park<S_H, true>(area_b, h1[nt][kc], pt0 + nt, kc, lane);
          ws_park<S_H, true>(area_b + P_H, dz[nt][kc], pt0 + nt, kc, lane);
        }
      layer_nt<T, NT, MT_H, 2, 0>(acc, dz, t_hid, nullptr, lane);  // dh1 = W_hid^T dz2
      gates(h1);                                                   // dz1
      ws_barrier();  // announces {h1, dz2}
      // ---- section C: {dz1, x} ----
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int kc = 0; kc < 2; ++kc) ws_park<S_H, true>(area_c, dz[nt][kc], pt0 + nt, kc, lane);
#pragma unroll
        for (int kc = 0; kc < KC_IN; ++kc) ws_park<S_X, true>(area_c + P_H, in[nt][kc], pt0 + nt, kc, lane);
      }
      if (a.dx != nullptr) {
        layer_nt<T, NT, MT_I, 2, 0>(acc, dz, t_in, nullptr, lane);  // dx = W_in^T dz1
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT_I; ++mt) {
            buf_v2u o;
            if (XC == 1) { o[0] = pack2<F16>(acc[nt][mt][0], acc[nt][mt][1]); o[1] = pack2<F16>(acc[nt][mt][2], acc[nt][mt][3]); }
            else if (XC == 2) { o[0] = pack2<BF16>(acc[nt][mt][0], acc[nt][mt][1]); o[1] = pack2<BF16>(acc[nt][mt][2], acc[nt][mt][3]); }
            else { o[0] = pack2<T>(acc[nt][mt][0], acc[nt][mt][1]); o[1] = pack2<T>(acc[nt][mt][2], acc[nt][mt][3]); }
            __builtin_amdgcn_raw_buffer_store_b64(o, rs_dx, at(chunk, pt0 + nt, a.dx_stride, off_dx[mt]), 0, 0);
          }
      }
    }
    ws_barrier();  // announces {dz1, x} of the last round
  } else {
    // ------------------------------------------------------------------ gradient waves
    const int d = (wave - CH) & (WS_CHAIN - 1), half = (wave - CH) / WS_CHAIN;
    const bool has_out = MT_O == 4 || half == 0;
    const f32x4_t zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int t = 0; t < TILES; ++t) acc_dw[t] = zero4;
#pragma unroll
    for (int u = 0; u < NBIAS; ++u) acc_db[u] = 0.0f;
    const uint32_t* area_a = panels + (size_t)d * SH::WAVE_DWORDS;
    const uint32_t* area_b = area_a + SH::AREA_A;
    const uint32_t* area_c = area_b + SH::AREA_B;
    auto section_c = [&]() {  // dW_in += dz1^T x, rows 32 half ..
      constexpr int JC = JB < MT_I ? JB : MT_I;
#pragma unroll
      for (int j0 = 0; j0 < MT_I; j0 += JC) {
        Frag xb[JC];
#pragma unroll
        for (int j = 0; j < JC; ++j) xb[j] = ws_operand<S_X>(area_c + P_H, j0 + j, lane);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const Frag da = ws_operand<S_H>(area_c, 2 * half + i, lane);
#pragma unroll
          for (int j = 0; j < JC; ++j) acc_dw[SH::T_IN + i * MT_I + j0 + j] = mfma16<T>(da, xb[j], acc_dw[SH::T_IN + i * MT_I + j0 + j]);
          if constexpr (B) {
            if (j0 == 0) {
#pragma unroll
              for (int q = 0; q < 4; ++q) acc_db[i] = dot2_ones<T>(da.w[q], acc_db[i]);
            }
          }
        }
      }
    };
    for (int round = 0; round < rounds; ++round) {
      ws_barrier();
      if (round > 0) section_c();
      ws_barrier();
      if (has_out) {  // dW_out += dy^T h2
#pragma unroll
        for (int j0 = 0; j0 < MT_H; j0 += JB) {
          Frag hb[JB];
#pragma unroll
          for (int j = 0; j < JB; ++j) hb[j] = ws_operand<S_H>(area_a, j0 + j, lane);
#pragma unroll
          for (int i = 0; i < SH::RO; ++i) {
            const Frag da = ws_operand<S_Y>(area_a + P_H, MT_O == 4 ? 2 * half + i : 0, lane);
#pragma unroll
            for (int j = 0; j < JB; ++j) acc_dw[SH::T_OUT + i * MT_H + j0 + j] = mfma16<T>(da, hb[j], acc_dw[SH::T_OUT + i * MT_H + j0 + j]);
            if constexpr (B) {
              if (j0 == 0) {
#pragma unroll
                for (int q = 0; q < 4; ++q) acc_db[4 + i] = dot2_ones<T>(da.w[q], acc_db[4 + i]);
              }
            }
          }
        }
      }
      ws_barrier();
      {  // dW_hid += dz2^T h1
#pragma unroll
        for (int j0 = 0; j0 < MT_H; j0 += JB) {
          Frag hb[JB];
#pragma unroll
          for (int j = 0; j < JB; ++j) hb[j] = ws_operand<S_H>(area_b, j0 + j, lane);
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const Frag da = ws_operand<S_H>(area_b + P_H, 2 * half + i, lane);
#pragma unroll
            for (int j = 0; j < JB; ++j) acc_dw[SH::T_HID + i * MT_H + j0 + j] = mfma16<T>(da, hb[j], acc_dw[SH::T_HID + i * MT_H + j0 + j]);
            if constexpr (B) {
              if (j0 == 0) {
#pragma unroll
                for (int q = 0; q < 4; ++q) acc_db[2 + i] = dot2_ones<T>(da.w[q], acc_db[2 + i]);
              }
            }
          }
        }
      }
    }
    ws_barrier();
    section_c();
  }

  // ---- sum the tiles of the four chunks' gradient waves through LDS (panels and weights are dead), one half of the
  // output features at a time; every wave adds up and flushes its share ----
  // where the sums go: the caller's accumulators (atomic adds), or this workgroup's own slot (plain stores)
  const bool own = a.partials != nullptr;
  float* slot = own ? a.partials + (size_t)blockIdx.x * a.partial_stride : nullptr;
  float* p_dw_in = own ? slot : a.dw_in;
  float* p_dw_hid = own ? p_dw_in + a.d_hidden * a.d_in : a.dw_hid;
  float* p_dw_out = own ? p_dw_hid + a.d_hidden * a.d_hidden : a.dw_out;
  float* p_db_in = own ? p_dw_out + a.d_out * a.d_hidden : a.db_in;
  float* p_db_hid = own ? p_db_in + a.d_hidden : a.db_hid;
  float* p_db_out = own ? p_db_hid + a.d_hidden : a.db_out;
  f32x4_t* red = reinterpret_cast<f32x4_t*>(smem);                               // [WS_CHAIN][TILES][64]
  float* redb = reinterpret_cast<float*>(smem) + (size_t)WS_CHAIN * TILES * 256;  // [WS_CHAIN][NBIAS][64]
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    __syncthreads();
    if (!chain && (wave - CH) / WS_CHAIN == h) {
      const int d = (wave - CH) & (WS_CHAIN - 1);
#pragma unroll
      for (int t = 0; t < TILES; ++t) red[((size_t)d * TILES + t) * 64 + lane] = acc_dw[t];
#pragma unroll
      for (int u = 0; u < NBIAS; ++u) redb[((size_t)d * NBIAS + u) * 64 + lane] = acc_db[u];
    }
    __syncthreads();
    constexpr int T_LAST = TILES;
#pragma unroll
    for (int t = 0; t < T_LAST; ++t) {
      if (t % WAVES != wave) continue;
      if (t >= SH::T_OUT && MT_O != 4 && h != 0) continue;  // a 16-row dW_out was summed with half 0
      const f32x4_t* p = red + (size_t)t * 64 + lane;
      const f32x4_t v = (p[0] + p[(size_t)TILES * 64]) + (p[(size_t)2 * TILES * 64] + p[(size_t)3 * TILES * 64]);
      if (t < SH::T_HID) flush_dw_tile(p_dw_in, a.d_hidden, a.d_in, 2 * h + (t - SH::T_IN) / MT_I, (t - SH::T_IN) % MT_I, lane, v, own);
      else if (t < SH::T_OUT) flush_dw_tile(p_dw_hid, a.d_hidden, a.d_hidden, 2 * h + (t - SH::T_HID) / MT_H, (t - SH::T_HID) % MT_H, lane, v, own);
      else flush_dw_tile(p_dw_out, a.d_out, a.d_hidden, (MT_O == 4 ? 2 * h : 0) + (t - SH::T_OUT) / MT_H, (t - SH::T_OUT) % MT_H, lane, v, own);
    }
    if constexpr (B) {
#pragma unroll
      for (int u = 0; u < NBIAS; ++u) {
        if (u % WAVES != wave) continue;
        if (u >= 4 && MT_O != 4 && h != 0) continue;
        const float* p = redb + (size_t)u * 64 + lane;
        const float v = (p[0] + p[(size_t)NBIAS * 64]) + (p[(size_t)2 * NBIAS * 64] + p[(size_t)3 * NBIAS * 64]);
        if (u < 2) flush_db(p_db_in, a.d_hidden, 2 * h + u, lane, v, own);
        else if (u < 4) flush_db(p_db_hid, a.d_hidden, 2 * h + u - 2, lane, v, own);
        else flush_db(p_db_out, a.d_out, (MT_O == 4 ? 2 * h : 0) + u - 4, lane, v, own);
      }
    }
  }
}

}  // namespace nf
