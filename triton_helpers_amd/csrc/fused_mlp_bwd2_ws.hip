// Host side of the role-split one-hidden-layer backward (fused_mlp_bwd2_ws.h): the 64-wide shapes whose weight
// gradients do not fit one wave next to the rest of the backward (d_in or d_out above the decoder shape's 32 / 16).
#include "fused_mlp_bwd2_ws.h"

namespace nf {

template <typename T, int KIN, int OUTP, int CH = WS_CHAIN_WAVES>
static int launch_ws(const MlpArgs& a0, hipStream_t s, int* blocks_out) {
  MlpArgs a = a0;
  constexpr size_t LDS = WsShape<KIN, OUTP>::LDS;
  constexpr int WAVES = CH + WS_GRAD;
  a.waves = WAVES;
  a.x_vec = a.dy_vec = a.dx_vec = 1;
  const int64_t chunks = (a.rows + 31) / 32;
  int64_t blocks = (chunks + WS_CHAIN - 1) / WS_CHAIN;
  const int64_t cap = (int64_t)device_cus();
  if (blocks > cap) blocks = cap;
  if (blocks_out != nullptr) *blocks_out = (int)blocks;
  const bool b = a.db_in != nullptr || a.db_hid != nullptr || a.db_out != nullptr || a.b_in != nullptr || a.b_hid != nullptr;
  const void* kern = b ? (const void*)mlp_bwd2_ws_k<T, KIN, OUTP, 0, true, CH> : (const void*)mlp_bwd2_ws_k<T, KIN, OUTP, 0, false, CH>;
  const hipError_t ea = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
  if (ea != hipSuccess) return fail((int)ea, "hipFuncSetAttribute: %s", hipGetErrorString(ea));
  void* args[] = {(void*)&a};
  const hipError_t e = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(64 * WAVES), args, LDS, s);
  if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(mlp_bwd2, role split): %s", hipGetErrorString(e));
  return check_launch("mlp_bwd2 (role split)");
}

template <typename T>
static int dispatch_ws(const MlpArgs& a, hipStream_t s, int* blocks_out) {
  const bool wide_in = a.d_in > 32, wide_out = a.d_out > 16;
  if (wide_in && wide_out) return launch_ws<T, 64, 64>(a, s, blocks_out);
  if (wide_in) return launch_ws<T, 64, 16>(a, s, blocks_out);
  return launch_ws<T, 32, 64>(a, s, blocks_out);
}

// Covers depth 2, d_hidden 64, ReLU, x stored like the weights, 8-byte aligned rows, extents a buffer descriptor
// reaches, and d_in > 32 or d_out > 16 (the decoder shape has a kernel of its own).  *blocks_out: workgroups launched
// (with MlpArgs::partials set, each stores its sums into the slot of its index).
int launch_mlp_bwd2_ws(const MlpArgs& a, int dtype, hipStream_t s, bool* handled, int* blocks_out) {
  *handled = false;
  const auto rows8 = [](const void* p, int64_t stride) { return (uintptr_t)p % 8 == 0 && stride % 4 == 0; };
  const auto reach = [&](int64_t stride) { return rows_in_reach(a.rows, stride); };
  const bool shape = a.depth == 2 && a.d_hidden == 64 && a.d_in <= 64 && a.d_out <= 64 && (a.d_in > 32 || a.d_out > 16) &&
                     a.act == NF_ACT_RELU && a.in_act == NF_ACT_NONE && a.x_conv == 0;
  const bool aligned = a.d_in % 4 == 0 && a.d_out % 4 == 0 && rows8(a.x, a.x_stride) && rows8(a.dy, a.dy_stride) &&
                       (a.dx == nullptr || rows8(a.dx, a.dx_stride));
  const bool in_reach = reach(a.x_stride) && reach(a.dy_stride) && (a.dx == nullptr || reach(a.dx_stride));
  if (!(shape && aligned && in_reach)) return 0;
  *handled = true;
  return dtype == NF_BF16 ? dispatch_ws<BF16>(a, s, blocks_out) : dispatch_ws<F16>(a, s, blocks_out);
}

}  // namespace nf
