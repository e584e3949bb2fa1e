// The one-hidden-layer backward (mlp_bwd2_k, fused_mlp_bwd2_kernels.h) for the shape of neural-field decoders and of the
// benchmark -- d_in <= 32, d_hidden = 64, d_out <= 16, ReLU -- on eight waves per workgroup: two waves per SIMD, each
// within half the register file (32-row chunks, the operands of the weight-gradient products transposed through LDS
// instead of the matrix core, rows addressed through buffer descriptors, bias sums compiled out when no bias gradient
// is asked for).  Everything else stays on the four-wave kernels of fused_mlp_bwd2.hip.
#include "fused_mlp_bwd2_kernels.h"

namespace nf {

template <typename T>
static int launch2_w8(const MlpArgs& a0, hipStream_t s) {
  MlpArgs a = a0;
  constexpr int KIN = 32, HP = 64, OUTP = 16, NT = 2, WAVES = 8;
  constexpr int KC_O = 1, MT_H = HP / 16, MT_I = KIN / 16, MT_O = OUTP / 16;
  constexpr size_t W_BYTES = ((size_t)MT_H * (KIN / 32) + (size_t)MT_I * (HP / 32) + 2 * (size_t)MT_H * (HP / 32) + (size_t)MT_H * KC_O) * 1024 +
                             (size_t)2 * HP * 4;
  constexpr int TILES = MT_H * (MT_I + MT_H) + MT_O * MT_H, NBIAS = 2 * MT_H + MT_O;
  static_assert(bwd2_parallel_sum(TILES, NBIAS), "the eight-wave kernel closes through the parallel sum");
  constexpr size_t RED = 4 * ((size_t)TILES * 1024 + (size_t)NBIAS * 256);
  constexpr size_t PANELS = W_BYTES + (size_t)WAVES * NT * TR_PANEL_DWORDS * 4;
  constexpr size_t LDS = PANELS > RED ? PANELS : RED;
  static_assert(LDS <= 160 * 1024, "LDS budget");
  a.waves = WAVES;
  a.x_vec = a.dy_vec = a.dx_vec = 1;
  const int64_t chunks = (a.rows + 16 * NT - 1) / (16 * NT);
  int64_t blocks = (chunks + WAVES - 1) / WAVES;
  const int64_t cap = (int64_t)device_cus();
  if (blocks > cap) blocks = cap;
  constexpr int XC_OTHER = T::code == NF_BF16 ? 1 : 2;
  const bool db = a.db_in != nullptr || a.db_hid != nullptr || a.db_out != nullptr;
  const void* kern;
  if (a.x_conv == 0)
    kern = db ? (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, true, true, NT, 0, true, WAVES, true, true>
              : (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, true, true, NT, 0, true, WAVES, true, false>;
  else
    kern = db ? (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, true, true, NT, XC_OTHER, true, WAVES, true, true>
              : (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, true, true, NT, XC_OTHER, true, WAVES, true, false>;
  const hipError_t ea = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
  if (ea != hipSuccess) return fail((int)ea, "hipFuncSetAttribute: %s", hipGetErrorString(ea));
  void* args[] = {(void*)&a};
  const hipError_t e = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(64 * WAVES), args, LDS, s);
  if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(mlp_bwd2, eight waves): %s", hipGetErrorString(e));
  return check_launch("mlp_bwd2 (eight waves)");
}

int launch_mlp_bwd2_w8(const MlpArgs& a, int dtype, hipStream_t s, bool* handled) {
  *handled = false;
  const int xc_other = dtype == NF_BF16 ? 1 : 2;
  const auto rows8 = [](const void* p, int64_t stride) { return (uintptr_t)p % 8 == 0 && stride % 4 == 0; };
  const int64_t limit = ((int64_t)1 << 31) - 1;  // bytes a buffer descriptor's 32-bit offsets reach
  const bool shape = a.depth == 2 && a.d_hidden == 64 && a.d_in <= 32 && a.d_out <= 16 && a.act == NF_ACT_RELU && a.in_act == NF_ACT_NONE &&
                     (a.x_conv == 0 || a.x_conv == xc_other);
  const bool aligned = a.d_in % 4 == 0 && a.d_out % 4 == 0 && rows8(a.x, a.x_stride) && rows8(a.dy, a.dy_stride) &&
                       (a.dx == nullptr || rows8(a.dx, a.dx_stride));
  const bool in_reach = a.rows * a.x_stride * 2 <= limit && a.rows * a.dy_stride * 2 <= limit && (a.dx == nullptr || a.rows * a.dx_stride * 2 <= limit);
  if (!shape || !aligned || !in_reach) return 0;
  *handled = true;
  return dtype == NF_BF16 ? launch2_w8<BF16>(a, s) : launch2_w8<F16>(a, s);
}

}  // namespace nf
