// One Adam step over a stacked hash table and the float32 gradient table that nf_hash_encode_bwd accumulates.
//
// The reference has no optimiser; this is the natural neighbour of its scatter-add
// (triton_helpers/layers/hash_encoding/kernel.py:432, 636): the step reads the float32 gradient once, un-scales it (loss scaling), updates the float32 moments and the
// float32 master copy, writes the 16-bit (or float32) table the encoder gathers from, and clears the gradient for the
// next backward -- the separate zero-fill pass over the gradient table disappears.
//
// Arithmetic is torch.optim.Adam's (no amsgrad, L2 weight decay added to the gradient):
//   g = grad / grad_scale (+ weight_decay * p);  m = b1 m + (1 - b1) g;  v = b2 v + (1 - b2) g g
//   p -= (lr / (1 - b1^t)) * m / (sqrt(v) / sqrt(1 - b2^t) + eps)
// Loss-scaled fp16 training meets overflowed gradients (the binned backward marks the rows of such a level with NaN):
// with NF_ADAM_SKIP_NONFINITE an element whose gradient is inf or NaN keeps its parameter and moments (what a skipped
// step does for it), and *found_nonfinite, when given, is set so that the caller can lower its loss scale.
// A pure stream: 34 bytes per element with a master copy and a 16-bit table.
#include "nf_common.h"

namespace nf {

template <typename TT, bool MASTER>
__global__ __launch_bounds__(256) void table_adam_k(typename TT::storage* table, float* master, float* grad, float* m, float* v,
                                                    int64_t n, float step_size, float inv_sqrt_bc2, float b1, float b2, float eps,
                                                    float weight_decay, float inv_scale, int flags, int* found_nonfinite) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    float p = MASTER ? master[i] : TT::to_f32(table[i]);
    float g = grad[i] * inv_scale;
    if (!(fabsf(g) <= 3.4028234e38f)) {  // inf or NaN
      if (found_nonfinite != nullptr) *found_nonfinite = 1;
      if (flags & NF_ADAM_SKIP_NONFINITE) {
        if (flags & NF_ADAM_CLEAR_GRAD) grad[i] = 0.0f;
        continue;
      }
    }
    if (weight_decay != 0.0f) g = fmaf(weight_decay, p, g);
    const float mi = fmaf(b1, m[i], (1.0f - b1) * g);
    const float vi = fmaf(b2, v[i], (1.0f - b2) * g * g);
    const float denom = sqrtf(vi) * inv_sqrt_bc2 + eps;
    p = p - step_size * (mi / denom);
    m[i] = mi;
    v[i] = vi;
    if (MASTER) master[i] = p;
    table[i] = TT::from_f32(p);
    if (flags & NF_ADAM_CLEAR_GRAD) grad[i] = 0.0f;
  }
}

}  // namespace nf

using namespace nf;

extern "C" int nf_table_adam_step(void* table, int table_dtype, float* master, float* grad, float* exp_avg, float* exp_avg_sq,
                                  int64_t n_elems, int64_t step, float lr, float beta1, float beta2, float eps, float weight_decay,
                                  float grad_scale, int flags, int* found_nonfinite, void* stream) {
  NF_REQUIRE(dtype_ok(table_dtype), NF_EINVAL, "unknown dtype code %d", table_dtype);
  NF_REQUIRE(n_elems >= 0, NF_EINVAL, "n_elems negative");
  NF_REQUIRE(step >= 1, NF_EINVAL, "step=%lld: steps count from 1", (long long)step);
  NF_REQUIRE(beta1 >= 0.0f && beta1 < 1.0f && beta2 >= 0.0f && beta2 < 1.0f, NF_EINVAL, "betas must lie in [0, 1)");
  NF_REQUIRE(eps >= 0.0f && grad_scale > 0.0f, NF_EINVAL, "eps must be >= 0 and grad_scale > 0");
  if (n_elems == 0) return 0;
  NF_REQUIRE(table && grad && exp_avg && exp_avg_sq, NF_EINVAL, "NULL pointer argument");
  const double bc1 = 1.0 - pow((double)beta1, (double)step), bc2 = 1.0 - pow((double)beta2, (double)step);
  const float step_size = (float)((double)lr / bc1), inv_sqrt_bc2 = (float)(1.0 / sqrt(bc2)), inv_scale = 1.0f / grad_scale;
  int64_t blocks = (n_elems + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;  // a grid-stride loop over the rest
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)blocks), block(256);
#define NF_ADAM_LAUNCH(TT)                                                                                                         \
  do {                                                                                                                             \
    if (master != nullptr)                                                                                                         \
      hipLaunchKernelGGL((table_adam_k<TT, true>), grid, block, 0, s, (TT::storage*)table, master, grad, exp_avg, exp_avg_sq, n_elems, \
                         step_size, inv_sqrt_bc2, beta1, beta2, eps, weight_decay, inv_scale, flags, found_nonfinite);          \
    else                                                                                                                           \
      hipLaunchKernelGGL((table_adam_k<TT, false>), grid, block, 0, s, (TT::storage*)table, master, grad, exp_avg, exp_avg_sq, n_elems, \
                         step_size, inv_sqrt_bc2, beta1, beta2, eps, weight_decay, inv_scale, flags, found_nonfinite);          \
  } while (0)
  if (table_dtype == NF_F32) NF_ADAM_LAUNCH(F32);
  else if (table_dtype == NF_F16) NF_ADAM_LAUNCH(F16);
  else NF_ADAM_LAUNCH(BF16);
#undef NF_ADAM_LAUNCH
  return check_launch("table_adam");
}
