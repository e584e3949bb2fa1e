// Host side of mlp_bwdn_k (fused_mlp_bwd2_kernels.h): ReLU nets of width 64 with two or three hidden-to-hidden layers.
#include "fused_mlp_bwd2_kernels.h"

namespace nf {

template <typename T, int KIN, int HP, int OUTP, int NH>
static int launchn(const MlpArgs& a0, hipStream_t s) {
  MlpArgs a = a0;
  constexpr int KC_O = (OUTP + 31) / 32;
  constexpr int MT_H = HP / 16, MT_I = KIN / 16, MT_O = OUTP / 16;
  constexpr size_t W_BYTES = ((size_t)MT_H * (KIN / 32) + (size_t)MT_I * (HP / 32) + 2 * (size_t)NH * MT_H * (HP / 32) + (size_t)MT_H * KC_O) * 1024 +
                             (size_t)(1 + NH) * HP * 4;
  constexpr int LA = bwdn_lds_layers(KIN, OUTP, NH);  // hidden accumulators kept in LDS, behind the weights
  constexpr size_t RED = (size_t)(MT_H * (MT_I + (NH - LA) * MT_H) + MT_O * MT_H) * 1024 + (size_t)((1 + NH) * MT_H + MT_O) * 256;
  constexpr size_t LDS = (W_BYTES > RED ? W_BYTES : RED) + (size_t)4 * LA * MT_H * MT_H * 1024;
  static_assert(LDS <= 160 * 1024, "LDS budget");
  a.waves = 4;
  a.x_vec = ((uintptr_t)a.x % 8 == 0) && (a.x_stride % 4 == 0);
  a.dy_vec = ((uintptr_t)a.dy % 8 == 0) && (a.dy_stride % 4 == 0);
  const int64_t chunks = (a.rows + 31) / 32;
  int64_t blocks = (chunks + 3) / 4;
  const int64_t cap = (int64_t)device_cus();
  if (blocks > cap) blocks = cap;
  const bool fast = a.x_vec && a.dy_vec && a.d_in % 4 == 0 && a.d_out % 4 == 0 &&
                    (a.dx == nullptr || ((uintptr_t)a.dx % 8 == 0 && a.dx_stride % 4 == 0));
  const void* kern;
  if constexpr (KIN == HP) {  // a layer in front has the hidden width
    kern = a.in_act != NF_ACT_NONE
               ? (fast ? (const void*)mlp_bwdn_k<T, KIN, HP, OUTP, NH, true, true> : (const void*)mlp_bwdn_k<T, KIN, HP, OUTP, NH, false, true>)
               : (fast ? (const void*)mlp_bwdn_k<T, KIN, HP, OUTP, NH, true, false> : (const void*)mlp_bwdn_k<T, KIN, HP, OUTP, NH, false, false>);
  } else {
    NF_REQUIRE(a.in_act == NF_ACT_NONE, NF_EUNSUPPORTED, "input activation with d_in=%d", a.d_in);
    kern = fast ? (const void*)mlp_bwdn_k<T, KIN, HP, OUTP, NH, true, false> : (const void*)mlp_bwdn_k<T, KIN, HP, OUTP, NH, false, false>;
  }
  if (LDS > 64 * 1024) {
    const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  void* args[] = {(void*)&a};
  const hipError_t e = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(256), args, LDS, s);
  if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(mlp_bwdn): %s", hipGetErrorString(e));
  return check_launch("mlp_bwdn");
}

template <typename T, int NH>
static int dispatchn(const MlpArgs& a, hipStream_t s) {
  const int kin = (a.d_in + 31) / 32 * 32, outp = a.d_out <= 16 ? 16 : 64;
  if (kin == 32 && outp == 16) return launchn<T, 32, 64, 16, NH>(a, s);
  if (kin == 32) return launchn<T, 32, 64, 64, NH>(a, s);
  if (outp == 16) return launchn<T, 64, 64, 16, NH>(a, s);
  return launchn<T, 64, 64, 64, NH>(a, s);
}

int launch_mlp_bwdn(const MlpArgs& a, int dtype, hipStream_t s, bool* handled) {
  *handled = false;
  // two hidden-to-hidden layers: the register-resident kernel covers wide ReLU nets with x in the parameters' dtype
  if (a.depth == 3 && a.d_hidden > 32 && a.act == NF_ACT_RELU && a.x_conv == 0) {
    *handled = true;
    return dtype == NF_BF16 ? dispatchn<BF16, 2>(a, s) : dispatchn<F16, 2>(a, s);
  }
  if (a.depth == 4 && a.d_hidden > 32 && a.act == NF_ACT_RELU && a.x_conv == 0) {
    *handled = true;
    return dtype == NF_BF16 ? dispatchn<BF16, 3>(a, s) : dispatchn<F16, 3>(a, s);
  }
  return 0;
}

}  // namespace nf
