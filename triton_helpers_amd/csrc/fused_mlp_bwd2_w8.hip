// The one-hidden-layer backward (mlp_bwd2_k, fused_mlp_bwd2_kernels.h) for the shape of neural-field decoders and of the
// benchmark -- d_in <= 32, d_hidden = 64, d_out <= 16, ReLU -- on eight waves per workgroup: two waves per SIMD, each
// within half the register file (32-row chunks, the operands of the weight-gradient products transposed through LDS
// instead of the matrix core, rows addressed through buffer descriptors, bias sums compiled out when no bias gradient
// is asked for).  Everything else stays on the four-wave kernels of fused_mlp_bwd2.hip.
#include "fused_mlp_bwd2_kernels.h"

namespace nf {

constexpr int ROUNDED_SLOTS = 512;  // most workgroups of a launch whose sums go to slots of their own

static size_t slot_floats(int d_in, int d_hidden, int d_out) {
  const size_t n = (size_t)d_hidden * d_in + (size_t)d_hidden * d_hidden + (size_t)d_out * d_hidden + 2 * (size_t)d_hidden + d_out;
  return (n + 63) / 64 * 64;
}

size_t mlp_bwd2_w8_rounded_bytes(int d_in, int d_hidden, int d_out) {
  return (size_t)ROUNDED_SLOTS * slot_floats(d_in, d_hidden, d_out) * sizeof(float);
}

struct RoundedPieces {
  void* out[6];      // dw_in, dw_hid, dw_out, db_in, db_hid, db_out (slot order); NULL: not wanted
  int first[7];      // first element of each piece inside a slot; first[6] = all
};

// out[piece][i] = round(sum over the workgroups' slots), the slots added in a fixed order: the same bits on every run
template <typename T>
__global__ __launch_bounds__(1024) void mlp_sum_slots_k(const float* partials, int n_slots, int64_t slot_stride, RoundedPieces pc) {
  __shared__ float part[16][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + tx;
  // sixteen interleaved runs over the slots (eight loads in flight each), then a fixed tree
  float sum = 0.0f;
  if (i < pc.first[6]) {
    int sl = ty;
    for (; sl + 112 < n_slots; sl += 128) {
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = partials[(size_t)(sl + 16 * k) * slot_stride + i];
#pragma unroll
      for (int k = 0; k < 8; ++k) sum += v[k];
    }
    for (; sl < n_slots; sl += 16) sum += partials[(size_t)sl * slot_stride + i];
  }
  part[ty][tx] = sum;
  __syncthreads();
  if (ty != 0 || i >= pc.first[6]) return;
  float total = 0.0f;
#pragma unroll
  for (int q = 0; q < 16; q += 4) total += (part[q][tx] + part[q + 1][tx]) + (part[q + 2][tx] + part[q + 3][tx]);
  int k = 0;
#pragma unroll
  for (int q = 1; q < 6; ++q) k += i >= pc.first[q];
  if (pc.out[k] != nullptr) reinterpret_cast<uint16_t*>(pc.out[k])[i - pc.first[k]] = T::from_f32(total);
}

template <typename T>
static int launch2_w8(const MlpArgs& a0, hipStream_t s, int* blocks_out = nullptr) {
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
  int64_t cap = (int64_t)device_cus();
  if (a.partials != nullptr && cap > ROUNDED_SLOTS) cap = ROUNDED_SLOTS;
  if (blocks > cap) blocks = cap;
  if (blocks_out != nullptr) *blocks_out = (int)blocks;
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

static bool w8_shape(const MlpArgs& a, int dtype) {
  const int xc_other = dtype == NF_BF16 ? 1 : 2;
  const auto rows8 = [](const void* p, int64_t stride) { return (uintptr_t)p % 8 == 0 && stride % 4 == 0; };
  const bool shape = a.depth == 2 && a.d_hidden == 64 && a.d_in <= 32 && a.d_out <= 16 && a.act == NF_ACT_RELU && a.in_act == NF_ACT_NONE &&
                     (a.x_conv == 0 || a.x_conv == xc_other);
  const bool aligned = a.d_in % 4 == 0 && a.d_out % 4 == 0 && rows8(a.x, a.x_stride) && rows8(a.dy, a.dy_stride) &&
                       (a.dx == nullptr || rows8(a.dx, a.dx_stride));
  const bool in_reach = rows_in_reach(a.rows, a.x_stride) && rows_in_reach(a.rows, a.dy_stride) && (a.dx == nullptr || rows_in_reach(a.rows, a.dx_stride));
  return shape && aligned && in_reach;
}

int launch_mlp_bwd2_w8(const MlpArgs& a, int dtype, hipStream_t s, bool* handled) {
  *handled = false;
  if (!w8_shape(a, dtype)) return 0;
  *handled = true;
  return dtype == NF_BF16 ? launch2_w8<BF16>(a, s) : launch2_w8<F16>(a, s);
}

int launch_mlp_bwd2_w8_rounded(const MlpArgs& a0, int dtype, void* const out[6], void* workspace, hipStream_t s, bool* handled) {
  *handled = false;
  const bool decoder = w8_shape(a0, dtype);
  MlpArgs a = a0;
  const size_t stride = slot_floats(a.d_in, a.d_hidden, a.d_out);
  a.partials = reinterpret_cast<float*>(workspace);
  a.partial_stride = (int64_t)stride;
  // bias sums are computed when any bias gradient is wanted (the kernel variant is chosen by these pointers)
  float* const any = a.partials;
  a.dw_in = a.dw_hid = a.dw_out = any;
  a.db_in = out[1] ? any : nullptr;
  a.db_hid = out[3] ? any : nullptr;
  a.db_out = out[5] ? any : nullptr;
  int blocks = 0;
  if (decoder) {
    *handled = true;
    if (int rc = dtype == NF_BF16 ? launch2_w8<BF16>(a, s, &blocks) : launch2_w8<F16>(a, s, &blocks)) return rc;
  } else {
    // the 64-wide inputs / outputs: chain and gradient waves, at most one workgroup per CU (fewer than ROUNDED_SLOTS)
    const int rc = launch_mlp_bwd2_ws(a, dtype, s, handled, &blocks);
    if (rc != 0 || !*handled) return rc;
  }
  RoundedPieces pc;
  const int H = a.d_hidden;
  const int sizes[6] = {H * a.d_in, H * H, a.d_out * H, H, H, a.d_out};
  void* const outs[6] = {out[0], out[2], out[4], out[1], out[3], out[5]};  // slot order: the three dW, then the three db
  int at = 0;
  for (int k = 0; k < 6; ++k) {
    pc.first[k] = at;
    pc.out[k] = outs[k];
    at += sizes[k];
  }
  pc.first[6] = at;
  const float* part = a.partials;
  const int64_t st = a.partial_stride;
  void* args[] = {(void*)&part, (void*)&blocks, (void*)&st, (void*)&pc};
  const void* kern = dtype == NF_BF16 ? (const void*)mlp_sum_slots_k<BF16> : (const void*)mlp_sum_slots_k<F16>;
  const hipError_t e = hipLaunchKernel(kern, dim3((unsigned)((at + 63) / 64)), dim3(1024), args, 0, s);
  if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(mlp_sum_slots): %s", hipGetErrorString(e));
  return check_launch("mlp_sum_slots");
}

}  // namespace nf
