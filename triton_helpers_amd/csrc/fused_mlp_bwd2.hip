// Host side of the fused-MLP backward kernels of fused_mlp_bwd2_kernels.h: shape dispatch and launches.
#include "fused_mlp_bwd2_kernels.h"

namespace nf {

template <typename T, int KIN, int HP, int OUTP>
static int launch2(const MlpArgs& a0, hipStream_t s) {
  MlpArgs a = a0;
  constexpr int KC_O = (OUTP + 31) / 32;
  constexpr int MT_H = HP / 16, MT_I = KIN / 16, MT_O = OUTP / 16;
  constexpr size_t W_BYTES = ((size_t)MT_H * (KIN / 32) + (size_t)MT_I * (HP / 32) + 2 * (size_t)MT_H * (HP / 32) + (size_t)MT_H * KC_O) * 1024 +
                             (size_t)2 * HP * 4;
  constexpr int TILES = MT_H * (MT_I + MT_H) + MT_O * MT_H, NBIAS = 2 * MT_H + MT_O;
  constexpr size_t RED = (bwd2_parallel_sum(TILES, NBIAS) ? 4 : 1) * ((size_t)TILES * 1024 + (size_t)NBIAS * 256);
  constexpr size_t LDS = W_BYTES > RED ? W_BYTES : RED;
  static_assert(LDS <= 160 * 1024, "LDS budget");
  a.waves = 4;
  // chain-order loads move 8 bytes at a time
  a.x_vec = ((uintptr_t)a.x % 8 == 0) && (a.x_stride % 4 == 0);
  a.dy_vec = ((uintptr_t)a.dy % 8 == 0) && (a.dy_stride % 4 == 0);
  // four tiles only where the registers allow it: ReLU (no gate images) and the narrow input / output shapes
  constexpr int NT = (KIN == 32 && OUTP == 16) ? NF_BWD2_NT : 2;
  const int nt = a.act == NF_ACT_RELU ? NT : 2;
  const int64_t chunks = (a.rows + 16 * nt - 1) / (16 * nt);
  int64_t blocks = (chunks + 3) / 4;
  const int64_t cap = (int64_t)device_cus() * (a.act == NF_ACT_RELU ? NF_BWD2_OCC : 1);
  if (blocks > cap) blocks = cap;
  const bool fast = a.x_vec && a.dy_vec && a.d_in % 4 == 0 && a.d_out % 4 == 0 &&
                    (a.dx == nullptr || ((uintptr_t)a.dx % 8 == 0 && a.dx_stride % 4 == 0));
  // x in the other 16-bit type: built for the aligned ReLU case only (the end-to-end encoder -> MLP step)
  constexpr int XC_OTHER = T::code == NF_BF16 ? 1 : 2;
  const void* kern;
  if (a.in_act != NF_ACT_NONE) {
    NF_REQUIRE(KIN == HP && a.x_conv == 0 && a.in_act == a.act, NF_EUNSUPPORTED, "input activation with d_in=%d", a.d_in);
    if constexpr (KIN == HP) {
      if (a.act == NF_ACT_RELU)
        kern = fast ? (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, true, true, NT, 3> : (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, true, false, NT, 3>;
      else
        kern = fast ? (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, false, true, 2, 3> : (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, false, false, 2, 3>;
    } else {
      return fail(NF_EUNSUPPORTED, "input activation with d_in=%d", a.d_in);
    }
  } else if (a.x_conv != 0) {
    NF_REQUIRE(fast && a.act == NF_ACT_RELU && a.x_conv == XC_OTHER, NF_EUNSUPPORTED,
               "x_dtype != dtype: the backward covers ReLU with 8-byte aligned rows only");
    kern = (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, true, true, NT, XC_OTHER>;
  } else if (a.act == NF_ACT_RELU) {
    kern = fast ? (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, true, true, NT, 0> : (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, true, false, NT, 0>;
  } else {
    kern = fast ? (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, false, true, 2, 0> : (const void*)mlp_bwd2_k<T, KIN, HP, OUTP, false, false, 2, 0>;
  }
  if (LDS > 64 * 1024) {
    const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  void* args[] = {(void*)&a};
  const hipError_t e = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(256), args, LDS, s);
  if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(mlp_bwd2): %s", hipGetErrorString(e));
  return check_launch("mlp_bwd2");
}

template <typename T>
static int dispatch2(const MlpArgs& a, hipStream_t s, bool* handled) {
  *handled = true;
  const int kin = (a.d_in + 31) / 32 * 32, outp = a.d_out <= 16 ? 16 : 64;
  if (a.d_hidden > 32) {
    if (kin == 32 && outp == 16) return launch2<T, 32, 64, 16>(a, s);
    if (kin == 32) return launch2<T, 32, 64, 64>(a, s);
    if (outp == 16) return launch2<T, 64, 64, 16>(a, s);
    return launch2<T, 64, 64, 64>(a, s);
  }
  *handled = false;  // narrow hidden layers stay on the general kernel
  return 0;
}

int launch_mlp_bwd2(const MlpArgs& a, int dtype, hipStream_t s, bool* handled) {
  *handled = false;
  if (a.depth == 2) {
    int rc = launch_mlp_bwd2_w8(a, dtype, s, handled);
    if (rc != 0 || *handled) return rc;
    rc = launch_mlp_bwd2_ws(a, dtype, s, handled);
    if (rc != 0 || *handled) return rc;
    return dtype == NF_BF16 ? dispatch2<BF16>(a, s, handled) : dispatch2<F16>(a, s, handled);
  }
  return launch_mlp_bwdn(a, dtype, s, handled);
}

}  // namespace nf
