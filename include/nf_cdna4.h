/*
 * nf_cdna4.h -- C ABI of libnf_cdna4.so: hand-written gfx950 (MI355X) kernels for
 * the three neural-field hot paths of triton_helpers.layers.
 *
 * Every entry point takes raw device pointers, sizes and strides in ELEMENTS,
 * dtype codes and a HIP stream handle (hipStream_t passed as void*; NULL = the
 * default stream).  Nothing is allocated, freed or synchronised inside the
 * library; work is enqueued on the given stream and the call returns.  All
 * functions return 0 on success, a negative NF_E* code on an argument error,
 * or a positive hipError_t; nf_last_error() returns a thread-local message.
 *
 * The functions replace the Triton launches of the reference (paths relative
 * to the reference repository):
 *   nf_hash_encode_fwd     <- _fwd_kernel[grid](...)   triton_helpers/layers/hash_encoding/kernel.py:575-590 (kernel :155-306)
 *   nf_hash_encode_bwd     <- _bwd_kernel[grid](...)   triton_helpers/layers/hash_encoding/kernel.py:641-656 (kernel :309-440)
 *   nf_hash_encode_indices <- embedding_lookup         triton_helpers/layers/hash_encoding/kernel.py:88-152
 *                             (exposed by the reference only through its test kernels,
 *                              tests/test_layers/test_hash_encoding.py:178-215)
 *   nf_mlp_fwd             <- _fwd_kernel[grid](...)   triton_helpers/layers/fully_fused_mlp/kernel.py:553-562 (kernel :181-261)
 *   nf_mlp_bwd             <- _bwd_kernel_rfs[grid](...) + host sum(0)
 *                                                      triton_helpers/layers/fully_fused_mlp/kernel.py:612-633 (kernel :307-500)
 *   nf_table_adam_step, nf_hash_encode_bwd_static, nf_hash_check_host : no counterpart (see their declarations)
 *   nf_revmlp_fwd / nf_revmlp_bwd : no counterpart in the reference (it has no
 *                             reversible MLP); same conventions as nf_mlp_*.
 */
#ifndef NF_CDNA4_H
#define NF_CDNA4_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NF_ABI_VERSION 9

/* element types */
enum { NF_F32 = 0, NF_F16 = 1, NF_BF16 = 2 };

/* activations (triton_helpers/ops.py:37-66; GELU = exact erf form, used by the reversible MLP) */
enum { NF_ACT_NONE = 0, NF_ACT_RELU = 1, NF_ACT_SILU = 2, NF_ACT_RELU2 = 3, NF_ACT_GELU = 4 };

/* error codes (negative) */
enum {
  NF_OK = 0,
  NF_EINVAL = -1,      /* bad argument value                           */
  NF_EUNSUPPORTED = -2,/* valid request this build has no kernel for    */
  NF_EALIGN = -3       /* pointer / stride alignment requirement unmet  */
};

#define NF_MAX_LEVELS 32
#define NF_MAX_DIMS 6

/* Level geometry of a hash encoding, computed on the host
 * (triton_helpers/layers/hash_encoding/helpers.py:26-115). */
typedef struct nf_hash_geom {
  int32_t dims;                 /* D, 1..NF_MAX_DIMS                                  */
  int32_t feat;                 /* F, features per table row                          */
  int32_t levels;               /* L, 1..NF_MAX_LEVELS                                */
  int32_t first_hash_level;     /* first level that hashes (>= levels: none)          */
  int64_t max_rows;             /* T, cap on rows per level                           */
  int32_t res[NF_MAX_LEVELS];   /* N_l                                                */
  int64_t rows[NF_MAX_LEVELS];  /* T_l = min((N_l+1)^D, T)                            */
  int64_t row_offset[NF_MAX_LEVELS]; /* first row of level l in the stacked table     */
} nf_hash_geom;

/* flags for the hash-encoding entry points */
enum {
  NF_HASH_FORCE_GENERIC = 1,   /* use the one-thread-per-(point,level) kernel even where a faster kernel applies */
  NF_HASH_FORCE_ATOMIC = 2,    /* backward: scatter with global atomics even where the LDS-tile kernels apply */
  NF_HASH_FORCE_PLANES = 4,    /* backward: of the two LDS-tile variants take the bit-plane one (smaller workspace) */
  NF_HASH_FWD_STAGED = 8,      /* forward: the LDS-staged tile kernel instead of the register-resident level sweep */
  NF_HASH_BWD_RECORDS = 16     /* backward: the sorted-record kernels even where a level is so few bins that the walk without records applies */
};

int nf_abi_version(void);
const char* nf_last_error(void);

/* out[n, l*F + f] = sum_j w_j(x_n, l) * table[row_offset[l] + row_j(x_n, l), f]
 * coords [n_points, D] (coords_dtype, strides in elements), coordinates in [0, scale];
 * table  [E, F] row-contiguous (table_dtype); out rows of table_dtype, row stride
 * out_stride_n elements (>= L*F; extra columns are left untouched);
 * primes: device pointer to >= D int64 hashing primes. */
int nf_hash_encode_fwd(const void* coords, int coords_dtype, int64_t coords_stride_n, int64_t coords_stride_d,
                       const void* table, int table_dtype, void* out, int64_t out_stride_n, int64_t n_points,
                       const nf_hash_geom* geom, const int64_t* primes, float scale, int flags, void* stream);

/* dtable[row_offset[l] + row_j, f] += w_j * dout[n, l*F + f]   (float32 accumulators,
 * NOT cleared by the call).  dout rows of dout_dtype with row stride dout_stride_n.
 * workspace: optional device scratch of at least nf_hash_encode_bwd_workspace_bytes() bytes (4-byte
 * aligned, 16-byte for the fastest variant); with it, large batches accumulate in LDS tiles instead of scattering
 * global atomics.
 * NULL / too small selects the atomic kernels.  Its contents are undefined afterwards. */
int nf_hash_encode_bwd(const void* coords, int coords_dtype, int64_t coords_stride_n, int64_t coords_stride_d,
                       const void* dout, int dout_dtype, int64_t dout_stride_n, float* dtable, int64_t n_points,
                       const nf_hash_geom* geom, const int64_t* primes, float scale, void* workspace,
                       int64_t workspace_bytes, int flags, void* stream);

/* Scratch bytes nf_hash_encode_bwd can use for this call shape and these flags (NF_HASH_FORCE_PLANES gives the
 * size of the smaller variant; tables of at most 2^14 rows per level take a walk without records and ask for
 * 4 bytes -- 8 with a float32 gradient -- per point, level and feature pair unless NF_HASH_BWD_RECORDS is set);
 * 0 when the workspace would not be used.
 * (No counterpart in the reference: its backward allocates nothing besides the gradient table,
 * triton_helpers/layers/hash_encoding/kernel.py:636.) */
int64_t nf_hash_encode_bwd_workspace_bytes(int64_t n_points, const nf_hash_geom* geom, int dout_dtype, int flags);

/* nf_hash_encode_bwd without the workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The
 * scratch of the sort-and-accumulate kernels is a device array inside the library, NF_HASH_BWD_STATIC_BYTES per GPU,
 * held until the process ends; the call allocates and frees nothing.  Batches whose scratch does not fit take the
 * smaller bit-plane variant where that applies (3-D points, 16-bit gradients: up to about 1.1 M points at L = 16) and
 * are refused with NF_EINVAL beyond that.  All calls on one GPU share the array: calls that overlap in time on one
 * GPU race on it.  The first call on a device resolves the array's address and sets the kernels' LDS attribute (it
 * may load the library's code object): make one warm-up call per device before recording calls into a HIP graph or
 * entering a region that may not touch the runtime's memory management.  Same arguments and results as
 * nf_hash_encode_bwd otherwise. */
#define NF_HASH_BWD_STATIC_BYTES (128 * 1024 * 1024)
int nf_hash_encode_bwd_static(const void* coords, int coords_dtype, int64_t coords_stride_n, int64_t coords_stride_d,
                              const void* dout, int dout_dtype, int64_t dout_stride_n, float* dtable, int64_t n_points,
                              const nf_hash_geom* geom, const int64_t* primes, float scale, int flags, void* stream);
int64_t nf_hash_encode_bwd_static_bytes(void);

/* Level-local table rows of all 2^D corners: out_rows [n_points, L, 2^D] int64, and
 * (optional, may be NULL) the interpolation weights out_w [n_points, L, 2^D] float32. */
int nf_hash_encode_indices(const void* coords, int coords_dtype, int64_t coords_stride_n, int64_t coords_stride_d,
                           int64_t* out_rows, float* out_w, int64_t n_points, const nf_hash_geom* geom,
                           const int64_t* primes, float scale, void* stream);

/* The same output computed with the index arithmetic of the fast kernels (the forward sweep / tiled kernels and the
 * binned backward): 32-bit wrap-around products and the level's mask instead of 64-bit products and a remainder.
 * D = 2 or 3, hashed levels with a power-of-two row count (NF_EUNSUPPORTED otherwise).  Same reference interface as
 * nf_hash_encode_indices (embedding_lookup, triton_helpers/layers/hash_encoding/kernel.py:88-152, whose device form
 * is this 32-bit one, :143-145); the two entry points must agree bit for bit. */
int nf_hash_encode_indices_fast(const void* coords, int coords_dtype, int64_t coords_stride_n, int64_t coords_stride_d,
                                int64_t* out_rows, float* out_w, int64_t n_points, const nf_hash_geom* geom,
                                const int64_t* primes, float scale, void* stream);

/* Host-side range check, the counterpart of the reference's debug-build asserts (tl.device_assert under
 * TRITON_DEBUG, triton_helpers/layers/hash_encoding/kernel.py:109-122, 151, 227-228).  Runs on the CPU, launches
 * nothing: coords is a HOST array [n_points, D] of float32 (row-contiguous), primes a HOST array of >= D values.
 * The kernels' own index functions are evaluated for every (point, level, corner); variant 0 is the 64-bit form of
 * the per-(point, level) kernels, variant 1 the 32-bit wrap-around form of the fast D = 2 / 3 kernels.
 * *n_bad_rows = corner rows >= rows[level] (cells are clamped to [0, N_l], so this is 0 for any input);
 * *n_bad_coords = coordinates outside [0, scale] or NaN (what the reference asserts);
 * rows_out (may be NULL): HOST array [n_points, L, 2^D] receiving the level-local rows. */
int nf_hash_check_host(const float* coords, int64_t n_points, const nf_hash_geom* geom, const int64_t* primes,
                       float scale, int variant, int64_t* rows_out, int64_t* n_bad_rows, int64_t* n_bad_coords);

/* One Adam step (torch.optim.Adam's arithmetic: no amsgrad, L2 weight decay) over a table of n_elems values and the
 * float32 gradient nf_hash_encode_bwd accumulated for it.  No counterpart in the reference, which ships no
 * optimiser: the natural neighbour of its scatter-add, triton_helpers/layers/hash_encoding/kernel.py:432, 636.
 * table [n_elems] in table_dtype; master: float32 copy of the parameters (NULL: the table itself is the parameter);
 * grad is divided by grad_scale (the loss scale) before use; exp_avg / exp_avg_sq: float32 moments; step counts from 1.
 * flags: NF_ADAM_CLEAR_GRAD zeroes grad for the next backward; NF_ADAM_SKIP_NONFINITE leaves the parameter and the
 * moments of an element untouched when its gradient is inf or NaN (an overflowed loss-scaled step; the binned backward
 * marks the rows of an overflowed level with NaN).  found_nonfinite (device int, may be NULL; cleared by the caller) is
 * set to 1 when any gradient element was inf or NaN, with or without the skip. */
#define NF_ADAM_CLEAR_GRAD 1
#define NF_ADAM_SKIP_NONFINITE 2
int nf_table_adam_step(void* table, int table_dtype, float* master, float* grad, float* exp_avg, float* exp_avg_sq,
                       int64_t n_elems, int64_t step, float lr, float beta1, float beta2, float eps, float weight_decay,
                       float grad_scale, int flags, int* found_nonfinite, void* stream);

/* Fully fused MLP.  x [rows, d_in] (row stride x_stride) in x_dtype, y [rows, d_out] (row stride y_stride) in `dtype`;
 * w_in [d_hidden, d_in], w_hid [(depth-1)*d_hidden, d_hidden], w_out [d_out, d_hidden], all
 * row-contiguous in `dtype`; biases b_in [d_hidden], b_hid [depth-1, d_hidden], b_out [d_out]
 * may each be NULL.  depth >= 1 counts the input layer plus the hidden layers.
 * dtype NF_F16 / NF_BF16: 16-bit operands, float32 accumulation (x_dtype may be the other 16-bit type).
 * dtype NF_F32 (x_dtype NF_F32 too): float32 storage, operands and accumulation (v_mfma_f32_16x16x4_f32) -- the
 * reference's float32 case, fully_fused_mlp/kernel.py:17-47 (TF32 products there: same range, shorter mantissa). */
int nf_mlp_fwd(const void* x, int64_t x_stride, void* y, int64_t y_stride, const void* w_in, const void* b_in,
               const void* w_hid, const void* b_hid, const void* w_out, const void* b_out, int64_t rows, int d_in,
               int d_hidden, int d_out, int depth, int act, int dtype, int x_dtype, void* workspace,
               int64_t workspace_bytes, void* stream);

/* Networks deeper than one launch holds on chip (forward: about 18 layers at d_hidden = 64; backward: 4 hidden-to-
 * hidden layers with ReLU at d_hidden = 64, 2 otherwise) run as a chain of
 * launches that hand 16-bit pre-activations [rows, d_hidden] to each other through `workspace` (16-byte aligned
 * device memory of at least this many bytes; contents are scratch).  0: one launch, workspace may be NULL.  Without
 * the workspace nf_mlp_bwd falls back to a slower one-launch kernel where the network fits it (NF_EINVAL otherwise).  (The
 * reference loops over the layers inside one kernel, triton_helpers/layers/fully_fused_mlp/kernel.py:139-178,
 * 264-304, re-reading every weight per program.)
 * dtype NF_F32: the forward needs none; the backward keeps every hidden layer's float32 pre-activation and always
 * needs depth * rows * d_hidden * 4 bytes plus 8.5 MB of partial weight gradients. */
int64_t nf_mlp_workspace_bytes(int64_t rows, int d_hidden, int depth, int act, int backward, int dtype);

/* x_dtype may be the other 16-bit type than `dtype` (an fp16 encoder output feeding bf16 weights): the rows are
 * converted while they are loaded, as a cast kernel in front would, and the backward writes dx in x_dtype.
 * nf_mlp_bwd takes a differing x_dtype for depth == 2, d_hidden > 32 (or depth == 1, d_hidden == 64), ReLU and 8-byte
 * aligned rows only (NF_EUNSUPPORTED otherwise).
 * depth == 1 (no hidden-to-hidden layer; w_hid, b_hid, dw_hid, db_hid NULL) with d_hidden == 64 and ReLU runs the
 * kernels of depth == 2 behind an identity layer that the library keeps on the device: after a ReLU, relu(I h) == h.
 *
 * Backward.  dx [rows, d_in] in x_dtype; the dw_ and db_ arguments are float32 accumulators shaped like the
 * weights/biases, NOT cleared by the call (db_* may be NULL; dx may be NULL). */
int nf_mlp_bwd(const void* x, int64_t x_stride, const void* dy, int64_t dy_stride, void* dx, int64_t dx_stride,
               const void* w_in, const void* b_in, const void* w_hid, const void* b_hid, const void* w_out,
               const void* b_out, float* dw_in, float* db_in, float* dw_hid, float* db_hid, float* dw_out,
               float* db_out, int64_t rows, int d_in, int d_hidden, int d_out, int depth, int act, int dtype,
               int x_dtype, void* workspace, int64_t workspace_bytes, void* stream);

/* nf_mlp_bwd with the weight and bias gradients delivered as the optimiser wants them: every dw_ / db_ buffer is in
 * `dtype`, and is WRITTEN with the sum over all rows, rounded once -- nothing to clear before the call and nothing to
 * cast after it (the reference's host-side sum(0) of per-program partials in the storage dtype,
 * triton_helpers/layers/fully_fused_mlp/kernel.py:627-633, in one place).  The workgroups' partial sums are added in a
 * fixed order, so the same inputs give the same bits on every run.  Built for depth == 2 (or depth == 1 with w_hid
 * and dw_hid NULL), d_hidden == 64, d_in <= 64, d_out <= 64 (both multiples of 4), ReLU, 8-byte aligned rows, and beyond
 * d_in 32 / d_out 16 x stored in `dtype`; NF_EUNSUPPORTED otherwise, before anything is launched.  workspace: 16-byte aligned, nf_mlp_bwd_rounded_workspace_bytes() bytes. */
int nf_mlp_bwd_rounded(const void* x, int64_t x_stride, const void* dy, int64_t dy_stride, void* dx, int64_t dx_stride,
                       const void* w_in, const void* b_in, const void* w_hid, const void* b_hid, const void* w_out,
                       const void* b_out, void* dw_in, void* db_in, void* dw_hid, void* db_hid, void* dw_out,
                       void* db_out, int64_t rows, int d_in, int d_hidden, int d_out, int depth, int act, int dtype,
                       int x_dtype, void* workspace, int64_t workspace_bytes, void* stream);
int64_t nf_mlp_bwd_rounded_workspace_bytes(int d_in, int d_hidden, int d_out);

/* Reversible MLP of `blocks` additive couplings over rows of width 2*half:
 *   y1 = x1 + F_k(x2),  y2 = x2 + G_k(y1),  F/G(u) = act(u W1^T + b1) W2^T + b2.
 * w1, w2 [blocks*2*half, half] (F_k then G_k per block), b1, b2 [blocks*2, half] or NULL. */
int nf_revmlp_fwd(const void* x, int64_t x_stride, void* y, int64_t y_stride, const void* w1, const void* b1,
                  const void* w2, const void* b2, int64_t rows, int half, int blocks, int act, int dtype,
                  void* stream);

/* Backward from the OUTPUT y: the inputs are recomputed block by block inside the kernel.
 * dx [rows, 2*half] in `dtype`; x_rec [rows, 2*half] in `dtype` (required: the kernel carries the stream between
 * couplings in it) receives the reconstructed input;
 * dw1, dw2, db1, db2 are float32 accumulators, NOT cleared by the call (db1, db2 may be NULL). */
int nf_revmlp_bwd(const void* y, int64_t y_stride, const void* dy, int64_t dy_stride, void* dx, int64_t dx_stride,
                  void* x_rec, int64_t x_rec_stride, const void* w1, const void* b1, const void* w2, const void* b2,
                  float* dw1, float* db1, float* dw2, float* db2, int64_t rows, int half, int blocks, int act,
                  int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NF_CDNA4_H */
