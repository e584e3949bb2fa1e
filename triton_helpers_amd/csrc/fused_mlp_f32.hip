// Fused MLP on float32 tensors with float32 products: v_mfma_f32_16x16x4_f32, float32 storage, operands and
// accumulation, so values keep the float32 range and 24-bit mantissa.  (The reference multiplies float32 tensors in
// TF32, fully_fused_mlp/kernel.py:17-47: the same range with a 10-bit mantissa.)  The 16-bit kernels are the fast
// path; this one is bound by the float32 matrix rate (157 TFLOP/s) and by its activations' round trip in the backward.
//
// Forward: one launch for any depth.  A wave carries 32 rows (two groups of 16) through all layers in registers.
// The product is formed transposed, out^T = W * h^T, so that the 16x16 result tile of a layer (lane (r, g), register v:
// feature 16*mt + 4*g + v of row r) is already the K operand of the next layer when K is walked in the order
// 16*t + 4*g + v; the weights are read from LDS in that order (one ds_read_b128 per four products).  Weights of all
// layers stay in LDS when they fit (up to eight layers), else each layer is staged in turn.
// Backward: the forward is replayed keeping every hidden layer's pre-activation in the caller's workspace
// ([depth][rows][d_hidden] float32), then one launch per layer, last to first, forms dW += dz^T h, db += sum dz and
// overwrites the pre-activation of the layer in front with its gradient.  A workgroup sums its waves' dW in LDS and
// stores one partial; a small second kernel adds the partials into the caller's accumulators (at most 32 adds per
// address: thousands of waves adding into the same 16 KB of dW directly cost more than the products).
#include "fused_mlp.h"

namespace nf {

constexpr int W32_STRIDE = 68;                           // floats per staged weight row (64 + 4)
constexpr int W32_LAYER = 64 * W32_STRIDE + 64;          // floats per staged layer: weights, then the bias
constexpr int W32_RESIDENT_MAX = 8;                      // layers kept in LDS at once
constexpr int T32_STRIDE = 80;                           // floats per row of a wave's 16-row transposing panel
constexpr int PART32 = 64 * 64 + 64;                     // floats of one workgroup's partial dW (64 x 64) and db (64)
constexpr int SLOTS32 = 512;                             // most workgroups of a backward launch
constexpr int NT32 = 2;                                  // 16-row groups a wave of the forward carries at once
constexpr int CHUNK32 = 4 * NT32 * 16;                   // rows per workgroup and pass of the forward

struct Mlp32Args {
  const float* x;
  int64_t x_stride;
  float* y;
  int64_t y_stride;
  const float *w_in, *b_in, *w_hid, *b_hid, *w_out, *b_out;
  float* z;  // [depth][rows][d_hidden] pre-activations, or NULL
  int64_t rows;
  int d_in, d_hidden, d_out, depth, act;
  int resident;  // 1: every layer's weights staged once per workgroup
  int n_layers;  // linear layers computed: depth + 1, or depth when only the pre-activations are wanted
};

__device__ __forceinline__ f32x4_t mfma4(float a, float b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// Rows x columns tile in "chain order": lane (r, g) holds columns 16*t + 4*g + v, v = 0..3, of row r.
__device__ __forceinline__ f32x4_t load_chain(const float* base, int64_t stride, int64_t row, int64_t rows, int col, int width,
                                              bool vec) {
  f32x4_t v = {0.0f, 0.0f, 0.0f, 0.0f};
  if (row >= rows) return v;
  const float* p = base + row * stride + col;
  if (vec && col + 3 < width) return *reinterpret_cast<const f32x4_t*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (col + i < width) v[i] = p[i];
  return v;
}

__device__ __forceinline__ void store_chain(float* base, int64_t stride, int64_t row, int64_t rows, int col, int width, bool vec,
                                            f32x4_t v) {
  if (row >= rows) return;
  float* p = base + row * stride + col;
  if (vec && col + 3 < width) {
    *reinterpret_cast<f32x4_t*>(p) = v;
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (col + i < width) p[i] = v[i];
}

__device__ __forceinline__ void stage_layer32(float* dst, const float* w, const float* b, int n_out, int n_in, int tid) {
  for (int i = tid; i < 64 * 64; i += 256) {
    const int o = i >> 6, c = i & 63;
    dst[o * W32_STRIDE + c] = (o < n_out && c < n_in) ? w[(size_t)o * n_in + c] : 0.0f;
  }
  if (tid < 64) dst[64 * W32_STRIDE + tid] = (b != nullptr && tid < n_out) ? b[tid] : 0.0f;
}

template <int ACT>
__global__ __launch_bounds__(256, 2) void mlp32_fwd_k(Mlp32Args a) {
  extern __shared__ float lds32[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int H = a.d_hidden, last = a.depth;
  auto layer_w = [&](int l) { return l == 0 ? a.w_in : l == last ? a.w_out : a.w_hid + (size_t)(l - 1) * H * H; };
  auto layer_b = [&](int l) -> const float* {
    return l == 0 ? a.b_in : l == last ? a.b_out : (a.b_hid ? a.b_hid + (size_t)(l - 1) * H : nullptr);
  };
  auto n_in = [&](int l) { return l == 0 ? a.d_in : H; };
  auto n_out = [&](int l) { return l == last ? a.d_out : H; };
  if (a.resident) {
    for (int l = 0; l < a.n_layers; ++l) stage_layer32(lds32 + l * W32_LAYER, layer_w(l), layer_b(l), n_out(l), n_in(l), tid);
    __syncthreads();
  }
  const bool x_vec = ((uintptr_t)a.x % 16 == 0) && (a.x_stride % 4 == 0);
  const bool y_vec = a.y != nullptr && ((uintptr_t)a.y % 16 == 0) && (a.y_stride % 4 == 0);
  const int64_t n_chunks = (a.rows + CHUNK32 - 1) / CHUNK32;
  for (int64_t chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
    const int64_t row0 = chunk * CHUNK32 + wave * (NT32 * 16) + r;
    f32x4_t h[NT32][4];
    const int kt_in = (a.d_in + 15) / 16;
#pragma unroll
    for (int nt = 0; nt < NT32; ++nt)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        h[nt][t] = t < kt_in ? load_chain(a.x, a.x_stride, row0 + 16 * nt, a.rows, 16 * t + 4 * g, a.d_in, x_vec)
                             : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    for (int l = 0; l < a.n_layers; ++l) {
      const float* wl = lds32;
      if (a.resident) {
        wl = lds32 + l * W32_LAYER;
      } else {
        __syncthreads();  // every wave is done with the layer before
        stage_layer32(lds32, layer_w(l), layer_b(l), n_out(l), n_in(l), tid);
        __syncthreads();
      }
      const int kt = (n_in(l) + 15) / 16, mt_n = (n_out(l) + 15) / 16;
      f32x4_t acc[NT32][4];
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
        const f32x4_t b4 = *reinterpret_cast<const f32x4_t*>(wl + 64 * W32_STRIDE + 16 * mt + 4 * g);
#pragma unroll
        for (int nt = 0; nt < NT32; ++nt) acc[nt][mt] = b4;
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        if (t >= kt) break;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
          if (mt >= mt_n) break;
          const f32x4_t w4 = *reinterpret_cast<const f32x4_t*>(wl + (16 * mt + r) * W32_STRIDE + 16 * t + 4 * g);
#pragma unroll
          for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int nt = 0; nt < NT32; ++nt) acc[nt][mt] = mfma4(w4[v], h[nt][t][v], acc[nt][mt]);
        }
      }
      if (l == last) {
#pragma unroll
        for (int nt = 0; nt < NT32; ++nt)
#pragma unroll
          for (int mt = 0; mt < 4; ++mt)
            if (mt < mt_n) store_chain(a.y, a.y_stride, row0 + 16 * nt, a.rows, 16 * mt + 4 * g, a.d_out, y_vec, acc[nt][mt]);
      } else {
#pragma unroll
        for (int nt = 0; nt < NT32; ++nt)
#pragma unroll
          for (int mt = 0; mt < 4; ++mt) {
            if (a.z != nullptr && mt < mt_n)
              store_chain(a.z + (size_t)l * a.rows * H, H, row0 + 16 * nt, a.rows, 16 * mt + 4 * g, H, true, acc[nt][mt]);
#pragma unroll
            for (int v = 0; v < 4; ++v) h[nt][mt][v] = mt < mt_n ? act_fwd(acc[nt][mt][v], ACT) : 0.0f;
          }
      }
    }
  }
}

struct Lin32BwdArgs {
  const float* dz;  // gradient at this layer's output (before the activation behind it), rows x n_out
  int64_t dz_stride;
  const float* src;  // this layer's input before its activation (rows x n_in): the layer in front's pre-activation, or x
  int64_t src_stride;
  float* dsrc;  // gradient at src (may be src itself, may be NULL)
  int64_t dsrc_stride;
  const float* w;  // n_out x n_in
  float* part;  // [gridDim.x][PART32] partial dW (row stride 64) and db of every workgroup
  int64_t rows;
  int n_out, n_in;
};

// One linear layer of the backward: partial dW = dz^T act(src), partial db = column sums of dz,
// dsrc = (dz W) * act'(src).
template <int ACT>
__global__ __launch_bounds__(256) void lin32_bwd_k(Lin32BwdArgs a) {
  extern __shared__ float lds32[];
  float* wt = lds32;  // wt[in][out], W32_STRIDE floats per row
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  float* pdz = lds32 + 64 * W32_STRIDE + wave * (2 * 16 * T32_STRIDE);  // this wave's dz rows
  float* ph = pdz + 16 * T32_STRIDE;                                    // this wave's act(src) rows
  for (int i = tid; i < 64 * 64; i += 256) {
    const int o = i >> 6, c = i & 63;
    wt[c * W32_STRIDE + o] = (o < a.n_out && c < a.n_in) ? a.w[(size_t)o * a.n_in + c] : 0.0f;
  }
  __syncthreads();
  const int mt_n = (a.n_out + 15) / 16, kt = (a.n_in + 15) / 16;
  const bool dz_vec = ((uintptr_t)a.dz % 16 == 0) && (a.dz_stride % 4 == 0);
  const bool src_vec = ((uintptr_t)a.src % 16 == 0) && (a.src_stride % 4 == 0);
  const bool dsrc_vec = a.dsrc != nullptr && ((uintptr_t)a.dsrc % 16 == 0) && (a.dsrc_stride % 4 == 0);
  f32x4_t dw[4][4];
  f32x4_t dbs[4];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    dbs[mt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) dw[mt][nt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  }
  const int64_t n_groups = (a.rows + 15) / 16;
  // the rows of the group after this one are asked for before this one's products (dsrc may be src itself: a group's
  // rows are read here before they are written, and no other wave touches them)
  auto load_group = [&](int64_t grp, f32x4_t (&dz)[4], f32x4_t (&z)[4]) {
    const int64_t row = grp * 16 + r;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      dz[t] = t < mt_n ? load_chain(a.dz, a.dz_stride, row, a.rows, 16 * t + 4 * g, a.n_out, dz_vec) : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
      z[t] = t < kt ? load_chain(a.src, a.src_stride, row, a.rows, 16 * t + 4 * g, a.n_in, src_vec) : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
  };
  const int64_t step = (int64_t)gridDim.x * 4;
  int64_t grp = (int64_t)blockIdx.x * 4 + wave;
  f32x4_t dz_next[4], z_next[4];
  if (grp < n_groups) load_group(grp, dz_next, z_next);
  for (; grp < n_groups; grp += step) {
    const int64_t row = grp * 16 + r;
    f32x4_t dz[4], z[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      dz[t] = dz_next[t];
      z[t] = z_next[t];
    }
    if (grp + step < n_groups) load_group(grp + step, dz_next, z_next);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      dbs[t] += dz[t];
      f32x4_t hv;
#pragma unroll
      for (int v = 0; v < 4; ++v) hv[v] = act_fwd(z[t][v], ACT);
      *reinterpret_cast<f32x4_t*>(pdz + r * T32_STRIDE + 16 * t + 4 * g) = dz[t];
      *reinterpret_cast<f32x4_t*>(ph + r * T32_STRIDE + 16 * t + 4 * g) = hv;
    }
    if (a.dsrc != nullptr) {
      // dsrc^T = W^T dz^T: rows of wt (input features) against the upstream gradient in chain order
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        if (nt >= kt) break;
        f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          if (t >= mt_n) break;
          const f32x4_t w4 = *reinterpret_cast<const f32x4_t*>(wt + (16 * nt + r) * W32_STRIDE + 16 * t + 4 * g);
#pragma unroll
          for (int v = 0; v < 4; ++v) acc = mfma4(w4[v], dz[t][v], acc);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[v] *= act_grad(z[nt][v], ACT);
        store_chain(a.dsrc, a.dsrc_stride, row, a.rows, 16 * nt + 4 * g, a.n_in, dsrc_vec, acc);
      }
    }
    // dW += dz^T h over this group's 16 rows, four rows per product; lane (i, k) reads row 4*s + k, column 16*tile + i
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      float bh[4];
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) bh[nt] = nt < kt ? ph[(4 * s + g) * T32_STRIDE + 16 * nt + r] : 0.0f;
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
        if (mt >= mt_n) break;
        const float av = pdz[(4 * s + g) * T32_STRIDE + 16 * mt + r];
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
          if (nt < kt) dw[mt][nt] = mfma4(av, bh[nt], dw[mt][nt]);
      }
    }
  }
  // the workgroup's four partial sums, added in wave order (the same result on every run), then one store
  __syncthreads();
  float* red = lds32;
  for (int w = 0; w < 4; ++w) {
    if (wave == w) {
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            float* p = red + (16 * mt + 4 * g + v) * 64 + 16 * nt + r;
            *p = w == 0 ? dw[mt][nt][v] : *p + dw[mt][nt][v];
          }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float sum = dbs[mt][v];
          sum += __shfl_xor(sum, 1);
          sum += __shfl_xor(sum, 2);
          sum += __shfl_xor(sum, 4);
          sum += __shfl_xor(sum, 8);
          float* p = red + 64 * 64 + 16 * mt + 4 * g + v;
          if (r == 0) *p = w == 0 ? sum : *p + sum;
        }
      }
    }
    __syncthreads();
  }
  for (int i = tid; i < PART32; i += 256) a.part[(size_t)blockIdx.x * PART32 + i] = red[i];
}

// dw += sum of the partial dW, db += sum of the partial db; blockIdx.y takes a share of the partials.
__global__ __launch_bounds__(256) void reduce32_k(const float* part, int n_slots, float* dw, float* db, int n_out, int n_in) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= PART32) return;
  const int per = (n_slots + gridDim.y - 1) / gridDim.y;
  const int s0 = blockIdx.y * per, s1 = min(n_slots, s0 + per);
  float sum = 0.0f;
  for (int sl = s0; sl < s1; ++sl) sum += part[(size_t)sl * PART32 + i];
  if (s0 >= s1) return;
  if (i < 64 * 64) {
    const int o = i >> 6, c = i & 63;
    if (o < n_out && c < n_in) unsafeAtomicAdd(dw + (size_t)o * n_in + c, sum);
  } else if (db != nullptr && i - 64 * 64 < n_out) {
    unsafeAtomicAdd(db + (i - 64 * 64), sum);
  }
}

template <typename Args>
static int launch32(const void* kern, const Args& a, int64_t blocks, size_t lds, hipStream_t s, const char* what) {
  if (lds > 64 * 1024) {
    const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  void* args[] = {(void*)&a};
  const hipError_t le = hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(256), args, lds, s);
  if (le != hipSuccess) return fail((int)le, "hipLaunchKernel(%s): %s", what, hipGetErrorString(le));
  return 0;
}

static int fwd32(Mlp32Args a, hipStream_t s) {
  a.n_layers = a.y != nullptr ? a.depth + 1 : a.depth;
  a.resident = a.n_layers <= W32_RESIDENT_MAX;
  const size_t lds = (size_t)(a.resident ? a.n_layers : 1) * W32_LAYER * sizeof(float);
  const int64_t chunks = (a.rows + CHUNK32 - 1) / CHUNK32;
  const int64_t cap = (int64_t)device_cus() * (lds > 76 * 1024 ? 1 : 2);
  const int64_t blocks = chunks < cap ? chunks : cap;
  const void* kern = nullptr;
  switch (a.act) {
    case NF_ACT_RELU: kern = (const void*)mlp32_fwd_k<NF_ACT_RELU>; break;
    case NF_ACT_SILU: kern = (const void*)mlp32_fwd_k<NF_ACT_SILU>; break;
    case NF_ACT_RELU2: kern = (const void*)mlp32_fwd_k<NF_ACT_RELU2>; break;
    case NF_ACT_GELU: kern = (const void*)mlp32_fwd_k<NF_ACT_GELU>; break;
    default: kern = (const void*)mlp32_fwd_k<NF_ACT_NONE>; break;
  }
  return launch32(kern, a, blocks, lds, s, "mlp32_fwd");
}

static int lin_bwd32(const Lin32BwdArgs& a, int act, float* dw, float* db, hipStream_t s) {
  const size_t lds = (size_t)(64 * W32_STRIDE + 4 * 2 * 16 * T32_STRIDE) * sizeof(float);
  const int64_t groups = (a.rows + 15) / 16;
  const int64_t want = (groups + 3) / 4;
  int64_t cap = (int64_t)device_cus() * 2;
  if (cap > SLOTS32) cap = SLOTS32;
  const int64_t blocks = want < cap ? want : cap;
  const void* kern = nullptr;
  switch (act) {
    case NF_ACT_RELU: kern = (const void*)lin32_bwd_k<NF_ACT_RELU>; break;
    case NF_ACT_SILU: kern = (const void*)lin32_bwd_k<NF_ACT_SILU>; break;
    case NF_ACT_RELU2: kern = (const void*)lin32_bwd_k<NF_ACT_RELU2>; break;
    case NF_ACT_GELU: kern = (const void*)lin32_bwd_k<NF_ACT_GELU>; break;
    default: kern = (const void*)lin32_bwd_k<NF_ACT_NONE>; break;
  }
  if (int rc = launch32(kern, a, blocks, lds, s, "lin32_bwd")) return rc;
  const float* part = a.part;
  int n_slots = (int)blocks, n_out = a.n_out, n_in = a.n_in;
  void* args[] = {(void*)&part, (void*)&n_slots, (void*)&dw, (void*)&db, (void*)&n_out, (void*)&n_in};
  const hipError_t le = hipLaunchKernel((const void*)reduce32_k, dim3((PART32 + 255) / 256, 32), dim3(256), args, 0, s);
  if (le != hipSuccess) return fail((int)le, "hipLaunchKernel(reduce32): %s", hipGetErrorString(le));
  return 0;
}

static size_t z32_bytes(int64_t rows, int d_hidden, int depth) {
  return ((size_t)depth * (size_t)rows * d_hidden * sizeof(float) + 255) / 256 * 256;
}

size_t mlp32_bwd_workspace_bytes(int64_t rows, int d_hidden, int depth) {
  return z32_bytes(rows, d_hidden, depth) + (size_t)SLOTS32 * PART32 * sizeof(float);
}

int mlp32_fwd(const float* x, int64_t x_stride, float* y, int64_t y_stride, const float* w_in, const float* b_in,
              const float* w_hid, const float* b_hid, const float* w_out, const float* b_out, int64_t rows, int d_in,
              int d_hidden, int d_out, int depth, int act, hipStream_t s) {
  Mlp32Args a = {};
  a.x = x; a.x_stride = x_stride; a.y = y; a.y_stride = y_stride;
  a.w_in = w_in; a.b_in = b_in; a.w_hid = w_hid; a.b_hid = b_hid; a.w_out = w_out; a.b_out = b_out;
  a.rows = rows; a.d_in = d_in; a.d_hidden = d_hidden; a.d_out = d_out; a.depth = depth; a.act = act;
  return fwd32(a, s);
}

int mlp32_bwd(const float* x, int64_t x_stride, const float* dy, int64_t dy_stride, float* dx, int64_t dx_stride,
              const float* w_in, const float* b_in, const float* w_hid, const float* b_hid, const float* w_out, float* dw_in,
              float* db_in, float* dw_hid, float* db_hid, float* dw_out, float* db_out, int64_t rows, int d_in, int d_hidden,
              int d_out, int depth, int act, void* workspace, int64_t workspace_bytes, hipStream_t s) {
  const size_t need = mlp32_bwd_workspace_bytes(rows, d_hidden, depth);
  NF_REQUIRE(workspace != nullptr && workspace_bytes >= (int64_t)need, NF_EINVAL,
             "float32 backward keeps %d pre-activations of %lld x %d float32 and partial weight gradients: it needs a "
             "workspace of %zu bytes (nf_mlp_workspace_bytes)", depth, (long long)rows, d_hidden, need);
  NF_REQUIRE((uintptr_t)workspace % 16 == 0, NF_EINVAL, "workspace must be 16-byte aligned");
  float* z = (float*)workspace;
  float* part = (float*)((char*)workspace + z32_bytes(rows, d_hidden, depth));
  const int H = d_hidden;
  Mlp32Args f = {};
  f.x = x; f.x_stride = x_stride; f.y = nullptr; f.y_stride = 0;
  f.w_in = w_in; f.b_in = b_in; f.w_hid = w_hid; f.b_hid = b_hid; f.w_out = w_out; f.b_out = nullptr;
  f.z = z;
  f.rows = rows; f.d_in = d_in; f.d_hidden = H; f.d_out = d_out; f.depth = depth; f.act = act;
  if (int rc = fwd32(f, s)) return rc;
  auto zl = [&](int l) { return z + (size_t)l * rows * H; };  // pre-activation of linear layer l, l < depth
  for (int l = depth; l >= 0; --l) {
    Lin32BwdArgs b = {};
    b.dz = l == depth ? dy : zl(l);
    b.dz_stride = l == depth ? dy_stride : H;
    b.src = l == 0 ? x : zl(l - 1);
    b.src_stride = l == 0 ? x_stride : H;
    b.dsrc = l == 0 ? dx : zl(l - 1);
    b.dsrc_stride = l == 0 ? dx_stride : H;
    b.w = l == 0 ? w_in : l == depth ? w_out : w_hid + (size_t)(l - 1) * H * H;
    float* dw = l == 0 ? dw_in : l == depth ? dw_out : dw_hid + (size_t)(l - 1) * H * H;
    float* db = l == 0 ? db_in : l == depth ? db_out : (db_hid ? db_hid + (size_t)(l - 1) * H : nullptr);
    b.part = part;
    b.rows = rows;
    b.n_out = l == depth ? d_out : H;
    b.n_in = l == 0 ? d_in : H;
    if (int rc = lin_bwd32(b, l == 0 ? NF_ACT_NONE : act, dw, db, s)) return rc;
  }
  return 0;
}

}  // namespace nf
