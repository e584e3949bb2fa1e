// Hash-encoding backward by binning (D = 2 or 3; features taken two at a time, the last one alone when their number is odd).
//
// Every (point, level, corner) contributes  w * dout[n, 2l .. 2l+1]  to one table row.  Scattering these with
// global atomics is bound by the chip's atomic request rate; accumulating them in LDS needs the contributions to
// one stretch of the table together.  So the contributions are first sorted by table bin (BIN_ROWS rows):
//
//   count   : per (level, bin) the number of records, for the whole batch (histogram) and per workgroup
//   offsets : exclusive scan of the histogram -> where each bin's records start; list of accumulation tasks
//   fill    : every workgroup takes FILL_POINTS points and, level by level, sorts their records by bin in LDS
//             and copies them out in runs, into room reserved with one atomic per (workgroup, bin)
//   accum   : one workgroup per (bin, slice of its records): the bin's rows live in LDS as two 64-bit integers
//             each and every contribution is one integer LDS atomic per feature (float LDS atomics and
//             compare-and-swap loops are an order of magnitude slower once a few thousand adds are in flight on
//             a tile); the tile is then converted and added to the gradient table (plain read-modify-write when
//             the bin has a single slice, atomics otherwise)
//
// A record is the pair of corners that differ in x only: 12 bytes {row0 | row1 << 13 inside the bin, w0 and w1 in
// 19-bit fixed point (rounded to nearest: each contribution is off by at most 2^-20 |dout|), packed 16-bit gradient
// pair}.  The records are written once and read once, 4 bytes less per record are worth more than the last bits of
// a weight.  The two rows of a pair share the bin: on a dense level they are
// neighbours, on a hashed level the x prime is 1 and  (x+1) ^ a  differs from  x ^ a  only below the lowest zero
// bit of x.  When they do not (bin border, 13 trailing ones in x) the pair becomes two records with one zero weight
// each.  The count and fill kernels apply the same rule, so their record counts agree.
//
// Dense levels whose cells span less than a bin (3-D, 16-bit gradients) take ONE record per point and level instead
// of four: {row of corner 0 relative to the bin, the three cell fractions in 18 / 16 / 16-bit fixed point, gradient
// pair}, still 12 bytes.  All eight corners lie within  res^2 + res + 1  rows of the first, so they fall into one bin
// or two neighbouring ones; a cell on a bin border is sent to both, and each accumulation takes the corners inside its
// own bin.  The accumulation rebuilds the eight trilinear weights from the fractions (each off by at most 2^-17).
//
// Integer accumulation: fill also finds max |dout| per level; with 2^e the power of two above it, a contribution
// w * g is accumulated as round(w * g * 2^(30 - e)), below 2^30 in magnitude, so a task's records cannot
// overflow 64 bits, the rounding is 2^-30 of the level's largest gradient per contribution, and a task's sum does
// not depend on the order of its records (tasks of a split bin still meet in float atomics).  A level whose gradient holds an inf or a nan gets nan in every row
// it touches.
//
// Arithmetic (cell, corner rows, weights) is the forward's, see hash_encoding.hip.
#include "hash_common.h"

namespace nf {

constexpr int BIN_ROWS_LOG2 = 13;
constexpr int BIN_ROWS = 1 << BIN_ROWS_LOG2;  // rows per bin (two 64-bit sums each: 128 KiB of LDS in the accumulation)
constexpr uint32_t BIN_MASK = BIN_ROWS - 1;
constexpr int W_BITS = 19;
constexpr uint32_t W_MAX = (1u << W_BITS) - 1u;
constexpr int FILL_POINTS = 1024;              // points (= threads) per workgroup of count and fill
constexpr int FILL_RECORDS = FILL_POINTS * 8; // most records a workgroup stages per level
constexpr int ACC_THREADS = 1024;
constexpr int ACC_INFLIGHT = 8;               // records in flight per thread
constexpr uint32_t SLICE_RECORDS = 98304;     // a bin with at most this many records is one accumulation task
constexpr uint32_t SPLIT_RECORDS = 32768;     // a bigger bin is cut into tasks of about this many
// A cell record stands for eight corners (sixteen LDS adds against an x-pair record's four).  In batches of up to
// CELL_FINE_MAX_POINTS points a cell level's tasks are cut four times finer: with the x-pair limits a coarse level of one
// or two bins was a single task of up to 98304 cell records, and from 2^16 to 2^17 points that one task (about 100 us)
// outlasted the rest of the accumulate launch (2^16 points: 109 -> 49 us, 2^17: 128 -> 57, 2^18: 89 -> 76).  Larger
// batches hide such a task behind the others, and four times as many flushes of the same few thousand rows cost them
// 30 us at 2^20 points.
constexpr uint32_t CELL_FINE = 4;
constexpr int64_t CELL_FINE_MAX_POINTS = (int64_t)1 << 18;
static uint32_t cell_task_div(int64_t n_points) { return n_points <= CELL_FINE_MAX_POINTS ? CELL_FINE : 1u; }
constexpr int MAX_BINS_PER_LEVEL = 2048;        // 2^24 rows
constexpr int MAX_BINS_TOTAL = 2560;          // LDS of the count and fill kernels

struct BinPlan {
  int n_levels;
  int nbins[NF_MAX_LEVELS];
  int binbase[NF_MAX_LEVELS + 1];  // first global bin of the level
  int cell[NF_MAX_LEVELS];         // the level's records are cells (one per point) instead of x-pairs
};

// cell record = {u | qx << 14,  qy | qz << 16,  packed gradient pair}: u = row of corner 0 minus the bin's first row,
// plus BIN_ROWS (the cell may start in the bin below); q* = the cell fractions in 18 / 16 / 16-bit fixed point
constexpr float CELL_QX = 262143.0f, CELL_QYZ = 65535.0f;
__device__ __forceinline__ uint3 make_cell_record(int32_t rel_row, const float (&fr)[3], uint32_t packed) {
  const uint32_t qx = (uint32_t)(fr[0] * CELL_QX + 0.5f), qy = (uint32_t)(fr[1] * CELL_QYZ + 0.5f), qz = (uint32_t)(fr[2] * CELL_QYZ + 0.5f);
  return make_uint3((uint32_t)(rel_row + BIN_ROWS) | qx << 14, qy | qz << 16, packed);
}

// workspace (32-bit words): hist[NB] | gmax[32] | cursor[NB] | n_tasks, pad[3] | tasks[max_tasks][4] |
// wg_counts[workgroups][NB] | records[R][3]      (hist and gmax are cleared together)
struct BinWs {
  uint32_t* hist;
  uint32_t* gmax;  // per level: largest |dout| bit pattern (15 bits)
  uint32_t* cursor;
  uint32_t* n_tasks;
  uint4* tasks;
  uint32_t* wg_counts;
  uint32_t* records;  // 3 words per record (16-bit gradient) or 4 (float32 gradient)
  uint32_t max_tasks;
};

// Workgroup barrier that orders LDS accesses only: global stores issued before it stay in flight (a plain
// __syncthreads() would wait for them to complete).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// record = {row0 | row1 << 13 | w1[18:13] << 26,  w0 | w1[12:0] << 19,  packed gradient pair}
__device__ __forceinline__ uint3 make_record(uint32_t row0, uint32_t row1, float w0, float w1, uint32_t packed) {
  const uint32_t q0 = (uint32_t)(w0 * (float)W_MAX + 0.5f), q1 = (uint32_t)(w1 * (float)W_MAX + 0.5f);
  return make_uint3(row0 | row1 << BIN_ROWS_LOG2 | (q1 >> 13) << 26, q0 | (q1 & 0x1fffu) << W_BITS, packed);
}

struct Located3 {
  uint32_t c[3];
  float fr[3];
};
template <int VD>
__device__ __forceinline__ Located3 locate(const float (&v)[VD], float fres) {
  Located3 r;
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    const float pos = v[d] * fres;
    const float fl = floorf(pos);
    r.c[d] = cell_index(fl, fres);
    r.fr[d] = pos - fl;
  }
  return r;
}
__device__ __forceinline__ void load_point(const void* coords, int cdt, int64_t csn, int64_t csd, int64_t n, float scale,
                                           float (&v)[3]) {
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    v[d] = load_as_f32(coords, n * csn + d * csd, cdt);
    if (scale != 1.0f) v[d] = v[d] / scale;
  }
}

// Dimensions beyond the third (sorted-record kernels, 4-D to 6-D points): a 4-D cell is its 3-D cell twice, once per
// corner of the fourth coordinate, so the 3-D pipeline runs once per such corner (`hi`, one bit per extra dimension).  The
// extra coordinates enter a pass as one term of the hash (xor), one of the dense index (add) and one factor of the weights.
struct ExtraDims {
  uint32_t hx;     // xor term of the 32-bit hash (hashed levels of a power of two of rows)
  uint64_t hx64;   // the same in 64 bits (hashed levels of any other size)
  uint32_t add;    // term of the dense index
  float w;         // factor of every corner weight
};
template <int DX, int VD>
__device__ __forceinline__ ExtraDims extra_dims(const float (&v)[VD], float fres, uint32_t res, int hi, const int64_t* primes) {
  static_assert(VD >= 3 + DX, "coordinate array too short");
  ExtraDims e = {0u, 0ull, 0u, 1.0f};
  uint32_t stride = res * res * res;
#pragma unroll
  for (int d = 0; d < DX; ++d) {
    const float pos = v[3 + d] * fres;
    const float fl = floorf(pos);
    const uint32_t bit = (uint32_t)(hi >> d) & 1u;
    const uint32_t c = cell_index(fl, fres) + bit;
    const float fr = pos - fl;
    e.hx ^= c * (uint32_t)primes[3 + d];
    e.hx64 ^= (uint64_t)c * (uint64_t)primes[3 + d];
    e.add += c * stride;
    stride *= res;
    const float wd = bit ? fr : 1.0f - fr;
    e.w = d == 0 ? wd : e.w * wd;
  }
  return e;
}

// Table rows (and trilinear / bilinear weights) of the 2^D corners of a point's cell, corner j = bit pattern of its
// offsets with x in bit 0, so that corners 2c and 2c+1 are an x-pair.  D = 3 or 2.
// A hashed level whose size is not a power of two takes the exact remainder of the 64-bit hash (the reference's
// CPU form) instead of the 32-bit wrap-around and mask.
template <int D, int VD>
__device__ __forceinline__ void cell_rows(const float (&v)[VD], float fres, bool hashed, uint32_t res, uint32_t mask,
                                          const uint32_t (&pi)[3], const int64_t* primes, uint32_t (&row)[1 << D], float* w,
                                          const ExtraDims* ex = nullptr) {
  const uint32_t n_rows = mask + 1u;
  if constexpr (D != 2 && D != 3) {
    // one, or more than three dimensions (the walk without records only): the per-(point, level) kernels' exact forms
    static_assert(VD >= D, "coordinate array too short");
    uint64_t p64[D];
#pragma unroll
    for (int d = 0; d < D; ++d) p64[d] = (uint64_t)primes[d];
    const Cell<D> cell = locate_cell<D>(v, (int)res);
#pragma unroll
    for (int j = 0; j < (1 << D); ++j) {
      const uint32_t r = (uint32_t)corner_row<D>(cell, j, hashed, res, n_rows, p64);
      row[j] = r < n_rows ? r : mask;  // (every row is inside its level; the tile that takes it is sized by the level)
      if (w != nullptr) w[j] = corner_weight<D>(cell, j);
    }
    return;
  } else {
  if (hashed && (n_rows & mask) != 0u) {
    uint32_t c[D];
    float fr[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const float pos = v[d] * fres;
      const float fl = floorf(pos);
      c[d] = cell_index(fl, fres);
      fr[d] = pos - fl;
    }
#pragma unroll
    for (int j = 0; j < (1 << D); ++j) {
      uint64_t h = 0;
#pragma unroll
      for (int d = 0; d < D; ++d) h ^= (uint64_t)(c[d] + ((j >> d) & 1)) * (uint64_t)primes[d];
      if (ex != nullptr) h ^= ex->hx64;
      row[j] = (uint32_t)(h % (uint64_t)n_rows);
    }
    if (w != nullptr) {
      if (D == 3) {
        weights_d3(fr, w);
        if (ex != nullptr)
#pragma unroll
          for (int j = 0; j < 8; ++j) w[j] = w[j] * ex->w;
      } else {
        const float gx = 1.0f - fr[0], gy = 1.0f - fr[1];
        w[0] = gx * gy;
        w[1] = fr[0] * gy;
        w[2] = gx * fr[1];
        w[3] = fr[0] * fr[1];
      }
    }
    return;
  }
  if (D == 3) {
    const Located3 q = locate(v, fres);
    const Corner8 r = rows_d3(q.c, hashed, res, mask, pi);
#pragma unroll
    for (int j = 0; j < (1 << D); ++j) row[j] = r.row[j];
    if (w != nullptr) weights_d3(q.fr, w);
    if (ex != nullptr) {
      // (a & m) ^ (b & m) == (a ^ b) & m: the extra xor term joins the masked rows; dense rows take the extra index term
      const uint32_t hx = ex->hx & mask;
#pragma unroll
      for (int j = 0; j < (1 << D); ++j) row[j] = hashed ? (row[j] ^ hx) : row[j] + ex->add;
      if (w != nullptr)
#pragma unroll
        for (int j = 0; j < (1 << D); ++j) w[j] = w[j] * ex->w;
    }
  } else {
    uint32_t c[2];
    float fr[2];
#pragma unroll
    for (int d = 0; d < 2; ++d) {
      const float pos = v[d] * fres;
      const float fl = floorf(pos);
      c[d] = cell_index(fl, fres);
      fr[d] = pos - fl;
    }
    if (hashed) {
      const uint32_t x0 = c[0] * pi[0], x1 = x0 + pi[0], y0 = c[1] * pi[1], y1 = y0 + pi[1];
      row[0] = (x0 ^ y0) & mask;
      row[1] = (x1 ^ y0) & mask;
      row[2] = (x0 ^ y1) & mask;
      row[3] = (x1 ^ y1) & mask;
    } else {
      const uint32_t b = c[0] + c[1] * res;
      row[0] = b;
      row[1] = b + 1;
      row[2] = b + res;
      row[3] = min(b + res + 1, mask);  // as in rows_d2: the zero-weight corner of x == scale stays inside the level
    }
    if (w != nullptr) {
      const float gx = 1.0f - fr[0], gy = 1.0f - fr[1];
      w[0] = gx * gy;
      w[1] = fr[0] * gy;
      w[2] = gx * fr[1];
      w[3] = fr[0] * fr[1];
    }
  }
  }
}
template <int D, int VD>
__device__ __forceinline__ void load_point_d(const void* coords, int cdt, int64_t csn, int64_t csd, int64_t n, float scale,
                                             float (&v)[VD]) {
#pragma unroll
  for (int d = 0; d < D; ++d) {
    v[d] = load_as_f32(coords, n * csn + d * csd, cdt);
    if (scale != 1.0f) v[d] = v[d] / scale;
  }
}

// Largest value of a wave, valid in lane 63: prefix maxima inside each row of 16 lanes, then lane 15 of rows 0 / 2 into
// rows 1 / 3 and lane 31 into rows 2 / 3 (data-parallel primitives of the vector ALU; nothing goes through LDS).
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t m) {
  auto step = [](uint32_t v, uint32_t shifted) { return shifted > v ? shifted : v; };
  m = step(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x111, 0xf, 0xf, false));  // row_shr:1
  m = step(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x112, 0xf, 0xf, false));  // row_shr:2
  m = step(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x114, 0xf, 0xf, false));  // row_shr:4
  m = step(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x118, 0xf, 0xf, false));  // row_shr:8
  m = step(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x142, 0xa, 0xf, false));  // row_bcast:15 -> rows 1, 3
  m = step(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x143, 0xc, 0xf, false));  // row_bcast:31 -> rows 2, 3
  return m;
}

__global__ void hash_bwd_bin_zero_k(uint32_t* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// ---------------------------------------------------------------------------------------
// count
// ---------------------------------------------------------------------------------------
// DX: dimensions beyond the third (D == 3 then); hi: which corner of them this pass covers
template <int D, int DX = 0>
__global__ __launch_bounds__(FILL_POINTS) void hash_bwd_bin_count_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                                    int64_t N, DevGeom g, BinPlan bp, const int64_t* primes,
                                                                    float scale, uint32_t* hist, uint32_t* wg_counts, int hi) {
  extern __shared__ uint32_t lh[];  // all bins of all levels
  const int tid = threadIdx.x, lane = tid & 63;
  const int NB = bp.binbase[bp.n_levels];
  for (int i = tid; i < NB; i += FILL_POINTS) lh[i] = 0u;
  lds_barrier();
  const int64_t n = (int64_t)blockIdx.x * FILL_POINTS + tid;
  const bool valid = n < N;
  float v[3 + DX] = {};
  constexpr int PAIRS = 1 << (D - 1);
  if (valid) load_point_d<D + DX>(coords, cdt, csn, csd, n, scale, v);
  const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], D > 2 ? (uint32_t)primes[D > 2 ? 2 : 0] : 0u};
  for (int l = 0; l < bp.n_levels; ++l) {
    uint32_t* cnt = lh + bp.binbase[l];
    const int nb = bp.nbins[l];
    const bool cells = D == 3 && bp.cell[l];
    if (nb == 1) {
      if (valid) {
        const unsigned long long m = __ballot(true);
        if (lane == __ffsll((long long)m) - 1) atomicAdd(cnt, (cells ? 1u : (uint32_t)PAIRS) * (uint32_t)__popcll(m));
      }
      continue;
    }
    if constexpr (D == 3) {
      if (cells) {
        // one record in the bin of corner 0 and, when the cell reaches into the next bin, one there
        const uint32_t res = (uint32_t)g.res[l];
        const Located3 q = locate(v, (float)g.res[l]);
        const uint32_t b = q.c[0] + q.c[1] * res + q.c[2] * res * res;
        const uint32_t k0 = b >> BIN_ROWS_LOG2, k1 = (b + res * res + res + 1u) >> BIN_ROWS_LOG2;
        if (valid) {
          atomicAdd(cnt + k0, 1u);
          if (k1 != k0) atomicAdd(cnt + k1, 1u);
        }
        continue;
      }
    }
    uint32_t row[1 << D];
    if constexpr (DX > 0) {
      const ExtraDims ex = extra_dims<DX>(v, (float)g.res[l], (uint32_t)g.res[l], hi, primes);
      cell_rows<D>(v, (float)g.res[l], l >= g.first_hash, (uint32_t)g.res[l], g.rows[l] - 1u, pi, primes, row, nullptr, &ex);
    } else {
      cell_rows<D>(v, (float)g.res[l], l >= g.first_hash, (uint32_t)g.res[l], g.rows[l] - 1u, pi, primes, row, nullptr);
    }
#pragma unroll
    for (int c = 0; c < PAIRS; ++c) {
      const uint32_t b0 = row[2 * c] >> BIN_ROWS_LOG2, b1 = row[2 * c + 1] >> BIN_ROWS_LOG2;
      if (valid) {
        atomicAdd(cnt + b0, 1u);
        if (b1 != b0) atomicAdd(cnt + b1, 1u);
      }
    }
  }
  lds_barrier();
  uint32_t* mine = wg_counts + (int64_t)blockIdx.x * NB;  // the fill kernel's workgroup of the same index reads these
  for (int i = tid; i < NB; i += FILL_POINTS) {
    const uint32_t c = lh[i];
    mine[i] = c;
    if (c) atomicAdd(hist + i, c);
  }
}

// ---------------------------------------------------------------------------------------
// offsets: one workgroup
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t x, uint32_t* wave_sums, uint32_t* total) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
  uint32_t incl = x;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t y = (uint32_t)__shfl_up((int)incl, d);
    if (lane >= d) incl += y;
  }
  __syncthreads();  // wave_sums may still be read from the previous call
  if (lane == 63) wave_sums[wave] = incl;
  __syncthreads();
  uint32_t before = 0, all = 0;
  for (int w = 0; w < nw; ++w) {
    const uint32_t s = wave_sums[w];
    if (w < wave) before += s;
    all += s;
  }
  *total = all;
  return before + incl - x;
}

__global__ __launch_bounds__(1024) void hash_bwd_bin_offsets_k(const uint32_t* hist, uint32_t* cursor, uint32_t* n_tasks,
                                                               uint4* tasks, int NB, uint32_t max_tasks, BinPlan bp,
                                                               uint32_t cell_div) {
  __shared__ uint32_t wave_sums[16];
  __shared__ uint32_t first_task[1025], bin_start[1024], bin_count[1024];  // of the 1024 bins of a pass
  uint32_t rec_run = 0, task_run = 0;
  for (int b0 = 0; b0 < NB; b0 += 1024) {
    const int b = b0 + (int)threadIdx.x;
    const uint32_t c = b < NB ? hist[b] : 0u;
    int lvl = 0;
    while (lvl + 1 < bp.n_levels && b >= bp.binbase[lvl + 1]) ++lvl;
    const bool cell = bp.cell[lvl] != 0;
    const uint32_t one = cell ? SLICE_RECORDS / cell_div : SLICE_RECORDS, cut = cell ? SPLIT_RECORDS / cell_div : SPLIT_RECORDS;
    const uint32_t slices = c <= one ? (c ? 1u : 0u) : (c + cut - 1u) / cut;
    uint32_t rec_total, task_total;
    const uint32_t start = rec_run + block_exclusive_scan(c, wave_sums, &rec_total);
    const uint32_t t0 = block_exclusive_scan(slices, wave_sums, &task_total);
    if (b < NB) cursor[b] = start;
    first_task[threadIdx.x] = t0;
    bin_start[threadIdx.x] = start;
    bin_count[threadIdx.x] = c;
    if (threadIdx.x == 0) first_task[1024] = task_total;
    __syncthreads();
    // every task of the pass by a thread of its own (a coarse dense level is one bin cut into a hundred slices): the
    // task's bin is the last one whose first task is not behind it
    for (uint32_t t = threadIdx.x; t < task_total; t += 1024) {
      uint32_t lo_b = 0, hi_b = 1023;
      while (lo_b < hi_b) {
        const uint32_t mid = (lo_b + hi_b + 1) >> 1;
        if (first_task[mid] <= t) lo_b = mid; else hi_b = mid - 1;
      }
      // bins without records share their first task with the bin behind them: the search lands on the last of the run
      const uint32_t c_b = bin_count[lo_b], n_sl = first_task[lo_b + 1] - first_task[lo_b], sl = t - first_task[lo_b];
      // equal slices, so that no workgroup gets a short tail
      const uint32_t per = (c_b + n_sl - 1u) / n_sl;
      uint32_t lo = bin_start[lo_b] + sl * per, hi = bin_start[lo_b] + (sl + 1u) * per;
      if (hi > bin_start[lo_b] + c_b) hi = bin_start[lo_b] + c_b;
      if (lo > hi) lo = hi;
      if (task_run + t < max_tasks) tasks[task_run + t] = make_uint4((uint32_t)b0 + lo_b, lo, hi, n_sl > 1u ? 1u : 0u);
    }
    __syncthreads();
    rec_run += rec_total;
    task_run += task_total;
  }
  if (threadIdx.x == 0) *n_tasks = task_run < max_tasks ? task_run : max_tasks;
}

// ---------------------------------------------------------------------------------------
// fill
// ---------------------------------------------------------------------------------------
// G32 = false: 16-bit upstream gradient, 12-byte records {.., .., packed pair}.  G32 = true: float32 upstream gradient,
// 16-byte records {.., .., g0, g1}; a staged entry then names the point instead of carrying the pair, and the copy-out
// takes the pair from the workgroup's per-level gradient table in LDS (the stage has no room for 20-byte entries).
template <bool G32, int D, int DX = 0>
__global__ __launch_bounds__(FILL_POINTS) void hash_bwd_bin_fill_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                                   const void* dout_v, int64_t dout_stride, int64_t N,
                                                                   DevGeom g, BinPlan bp, const int64_t* primes, float scale,
                                                                   const uint32_t* wg_counts, uint32_t* cursor, uint32_t* gmax,
                                                                   uint32_t* records_v, int feat, int f0, int hi) {
  extern __shared__ __align__(16) unsigned char fill_smem[];
  const int NB = bp.binbase[bp.n_levels];
  const uint16_t* dout = reinterpret_cast<const uint16_t*>(dout_v);
  uint3* records = reinterpret_cast<uint3*>(records_v);
  uint4* records4 = reinterpret_cast<uint4*>(records_v);
  uint4* stage = reinterpret_cast<uint4*>(fill_smem);                     // [FILL_RECORDS] {record, its place in `records`}, sorted by bin
  uint2* gtab = reinterpret_cast<uint2*>(stage + FILL_RECORDS);           // G32: [FILL_POINTS] this level's gradient pair of every point
  uint32_t* cur = reinterpret_cast<uint32_t*>(gtab + (G32 ? FILL_POINTS : 0));  // [NB] next staged position of a bin
  uint32_t* delta = cur + NB;                                             // [NB] global minus staged position
  uint32_t* totals = delta + NB;                                          // [levels] records of this workgroup per level
  uint32_t* lmax = totals + NF_MAX_LEVELS;                                // [levels] largest |dout| pattern
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t n0 = (int64_t)blockIdx.x * FILL_POINTS;
  const int64_t n = n0 + tid;
  const bool valid = n < N;
  // This workgroup's share of every bin, counted by the count kernel: one reservation per non-empty bin, all in
  // flight together.
  for (int i = tid; i < NB; i += FILL_POINTS) {
    const uint32_t c = wg_counts[(int64_t)blockIdx.x * NB + i];
    cur[i] = c;
    delta[i] = c ? atomicAdd(cursor + i, c) : 0u;
  }
  if (tid < NF_MAX_LEVELS) lmax[tid] = 0u;
  float v[3 + DX] = {};
  constexpr int PAIRS = 1 << (D - 1);
  if (valid) load_point_d<D + DX>(coords, cdt, csn, csd, n, scale, v);
  const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], D > 2 ? (uint32_t)primes[D > 2 ? 2 : 0] : 0u};
  // this point's gradient row, read once (up to 16 levels live in registers); float32 rows are read level by level
  const uint32_t* grow = reinterpret_cast<const uint32_t*>(dout + (valid ? n : 0) * dout_stride);
  const float* grow32 = reinterpret_cast<const float*>(dout_v) + (valid ? n : 0) * dout_stride;
  uint32_t gr[16];
  // this pass covers features f0, f0 + 1 of every level: the pair of level l sits at element l * feat + f0 of the row
  // (rows of 2, 4 or 8 features in 16-byte pieces: with 4 or 8 features a piece holds the pairs of two levels or of one,
  // and the pass keeps its own; per-level 4-byte reads touch a point's 128 or 256 bytes sixteen times instead)
  const bool row_vec = !G32 && (feat == 2 || feat == 4 || feat == 8) && bp.n_levels <= 16 && (bp.n_levels & 3) == 0 &&
                       ((uintptr_t)dout & 15u) == 0 && (dout_stride & 7) == 0;
  const bool row_vec32 = G32 && feat == 2 && (bp.n_levels & 3) == 0 && ((uintptr_t)dout_v & 15u) == 0 && (dout_stride & 3) == 0;
  uint2 held[3] = {make_uint2(0u, 0u), make_uint2(0u, 0u), make_uint2(0u, 0u)};
  const int pair_in_level = f0 >> 1;
  auto word = [](const uint4& q, int c) { return c == 0 ? q.x : c == 1 ? q.y : c == 2 ? q.z : q.w; };
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint4 t = make_uint4(0u, 0u, 0u, 0u);
    if (row_vec && valid && 4 * i < bp.n_levels) {
      const uint4* g4 = reinterpret_cast<const uint4*>(grow);
      if (feat == 2) {
        t = g4[i];
      } else if (feat == 4) {
        const uint4 a = g4[2 * i], b = g4[2 * i + 1];
        t = pair_in_level ? make_uint4(a.y, a.w, b.y, b.w) : make_uint4(a.x, a.z, b.x, b.z);
      } else {
        const uint4 q0 = g4[4 * i], q1 = g4[4 * i + 1], q2 = g4[4 * i + 2], q3 = g4[4 * i + 3];
        t = make_uint4(word(q0, pair_in_level), word(q1, pair_in_level), word(q2, pair_in_level), word(q3, pair_in_level));
      }
    }
    gr[4 * i] = t.x;
    gr[4 * i + 1] = t.y;
    gr[4 * i + 2] = t.z;
    gr[4 * i + 3] = t.w;
  }
  lds_barrier();
  // staged start of every bin inside its level (exclusive scan of the counts), one wave per level
  for (int l = wave; l < bp.n_levels; l += FILL_POINTS / 64) {
    const int nb = bp.nbins[l], gb0 = bp.binbase[l];
    uint32_t run = 0;
    for (int b0 = 0; b0 < nb; b0 += 64) {
      const int b = b0 + lane;
      const uint32_t c = b < nb ? cur[gb0 + b] : 0u;
      uint32_t incl = c;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t y = (uint32_t)__shfl_up((int)incl, d);
        if (lane >= d) incl += y;
      }
      const uint32_t excl = run + incl - c;
      if (b < nb) {
        cur[gb0 + b] = excl;
        delta[gb0 + b] -= excl;
      }
      run += (uint32_t)__shfl((int)incl, 63);
    }
    if (lane == 0) totals[l] = run;
  }
  lds_barrier();

  for (int l = 0; l < bp.n_levels; ++l) {
    const int nb = bp.nbins[l];
    uint32_t* lcur = cur + bp.binbase[l];
    const uint32_t* ldelta = delta + bp.binbase[l];
    uint32_t packed = 0u;  // 16-bit: the pair; float32: the point's index in the workgroup (its pair goes to gtab)
    if (G32) {
      uint2 pair = make_uint2(0u, 0u);
      if (valid) {
        if (feat & 1) {  // an odd row width: the pair is not 8-byte aligned, and the last feature has no partner
          pair.x = __float_as_uint(grow32[l * feat + f0]);
          if (f0 + 1 < feat) pair.y = __float_as_uint(grow32[l * feat + f0 + 1]);
        } else if (row_vec32) {  // four levels' pairs in two 16-byte reads: a quarter of the passes over the point's 128 bytes
          if ((l & 3) == 0) {
            const uint4 q0 = *reinterpret_cast<const uint4*>(grow32 + 2 * l), q1 = *reinterpret_cast<const uint4*>(grow32 + 2 * l + 4);
            pair = make_uint2(q0.x, q0.y);
            held[0] = make_uint2(q0.z, q0.w);
            held[1] = make_uint2(q1.x, q1.y);
            held[2] = make_uint2(q1.z, q1.w);
          } else {
            pair = (l & 3) == 1 ? held[0] : (l & 3) == 2 ? held[1] : held[2];
          }
        } else {
          pair = *reinterpret_cast<const uint2*>(grow32 + l * feat + f0);
        }
      }
      gtab[tid] = pair;
      packed = (uint32_t)tid;
      // largest |g| of the level: positive float patterns order like integers
      const uint32_t a0 = pair.x & 0x7fffffffu, a1 = pair.y & 0x7fffffffu;
      const uint32_t m = wave_max_u32(a0 > a1 ? a0 : a1);
      if (lane == 63 && m) atomicMax(lmax + l, m);
    } else {
      if (row_vec) {
        packed = gr[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) packed = (l == i) ? gr[i] : packed;
      } else if (valid) {
        if (feat & 1) {  // an odd row width: 16-bit loads, and the last feature has no partner
          const uint16_t* g16 = reinterpret_cast<const uint16_t*>(grow);
          packed = g16[l * feat + f0];
          if (f0 + 1 < feat) packed |= (uint32_t)g16[l * feat + f0 + 1] << 16;
        } else {
          packed = grow[(l * feat + f0) >> 1];
        }
      }
      // largest |g| of the level: positive 16-bit float patterns order like integers
      const uint32_t pk = packed & 0x7fff7fffu;
      const uint32_t m = wave_max_u32((pk & 0xffffu) > (pk >> 16) ? (pk & 0xffffu) : (pk >> 16));
      if (lane == 63 && m) atomicMax(lmax + l, m);
    }
    bool cells = false;
    if constexpr (D == 3 && !G32) cells = bp.cell[l] != 0;
    if (cells) {
      const uint32_t res = (uint32_t)g.res[l];
      const Located3 q = locate(v, (float)g.res[l]);
      const uint32_t b = q.c[0] + q.c[1] * res + q.c[2] * res * res;
      const uint32_t k0 = b >> BIN_ROWS_LOG2, k1 = (b + res * res + res + 1u) >> BIN_ROWS_LOG2;
      const bool two = k1 != k0;
      uint32_t pos0;
      if (nb == 1) pos0 = (uint32_t)tid;  // the valid points are the first of the workgroup
      else pos0 = valid ? atomicAdd(lcur + k0, 1u) : 0u;
      if (valid) {
        const uint3 rec = make_cell_record((int32_t)(b - (k0 << BIN_ROWS_LOG2)), q.fr, packed);
        stage[pos0] = make_uint4(rec.x, rec.y, rec.z, pos0 + ldelta[k0]);
      }
      if (nb > 1 && __any(valid && two)) {
        const bool on = valid && two;
        const uint32_t pos1 = on ? atomicAdd(lcur + k1, 1u) : 0u;
        if (on) {
          const uint3 rec = make_cell_record((int32_t)b - (int32_t)(k1 << BIN_ROWS_LOG2), q.fr, packed);
          stage[pos1] = make_uint4(rec.x, rec.y, rec.z, pos1 + ldelta[k1]);
        }
      }
    } else {
      uint32_t row[1 << D];
      float w[1 << D];
      if constexpr (DX > 0) {
        const ExtraDims ex = extra_dims<DX>(v, (float)g.res[l], (uint32_t)g.res[l], hi, primes);
        cell_rows<D>(v, (float)g.res[l], l >= g.first_hash, (uint32_t)g.res[l], g.rows[l] - 1u, pi, primes, row, w, &ex);
      } else {
        cell_rows<D>(v, (float)g.res[l], l >= g.first_hash, (uint32_t)g.res[l], g.rows[l] - 1u, pi, primes, row, w);
      }
      // The x-pairs of the point (four in 3-D, two in 2-D): their ranks are asked for together, so that a wave waits
      // for LDS once per level and not once per pair.
      uint32_t b0[PAIRS], b1[PAIRS], pos[PAIRS], dlt[PAIRS];
      bool split[PAIRS];
      bool any_split = false;
#pragma unroll
      for (int c = 0; c < PAIRS; ++c) {
        b0[c] = row[2 * c] >> BIN_ROWS_LOG2;
        b1[c] = row[2 * c + 1] >> BIN_ROWS_LOG2;
        split[c] = b1[c] != b0[c];
        any_split = any_split || split[c];
      }
      if (nb == 1) {
#pragma unroll
        for (int c = 0; c < PAIRS; ++c) pos[c] = (uint32_t)tid * (uint32_t)PAIRS + (uint32_t)c;  // the valid points are the first of the workgroup
      } else {
#pragma unroll
        for (int c = 0; c < PAIRS; ++c) pos[c] = valid ? atomicAdd(lcur + b0[c], 1u) : 0u;
      }
#pragma unroll
      for (int c = 0; c < PAIRS; ++c) dlt[c] = ldelta[b0[c]];
      if (valid) {
#pragma unroll
        for (int c = 0; c < PAIRS; ++c) {
          const uint32_t r0 = row[2 * c], r1 = row[2 * c + 1];
          const uint3 rec = make_record(r0 & BIN_MASK, (split[c] ? r0 : r1) & BIN_MASK, w[2 * c], split[c] ? 0.0f : w[2 * c + 1], packed);
          stage[pos[c]] = G32 ? make_uint4(rec.x, rec.y, pos[c] + dlt[c], rec.z) : make_uint4(rec.x, rec.y, rec.z, pos[c] + dlt[c]);
        }
      }
      // a pair that straddles two bins leaves its second corner as a record of its own (rare)
      if (nb > 1 && __any(valid && any_split)) {
#pragma unroll
        for (int c = 0; c < PAIRS; ++c) {
          const bool on = valid && split[c];
          if (!__any(on)) continue;
          const uint32_t pos1 = on ? atomicAdd(lcur + b1[c], 1u) : 0u;
          if (on) {
            const uint32_t r1 = row[2 * c + 1];
            const uint3 rec = make_record(r1 & BIN_MASK, r1 & BIN_MASK, w[2 * c + 1], 0.0f, packed);
            const uint32_t gp = pos1 + ldelta[b1[c]];
            stage[pos1] = G32 ? make_uint4(rec.x, rec.y, gp, rec.z) : make_uint4(rec.x, rec.y, rec.z, gp);
          }
        }
      }
    }
    lds_barrier();
    const uint32_t total = totals[l];
    for (uint32_t i = tid; i < total; i += FILL_POINTS) {
      const uint4 e = stage[i];
      if (G32) {
        const uint2 pair = gtab[e.w];
        records4[e.z] = make_uint4(e.x, e.y, pair.x, pair.y);
      } else {
        records[e.w] = make_uint3(e.x, e.y, e.z);
      }
    }
    lds_barrier();  // the next level overwrites the stage
  }
  if (tid < bp.n_levels) {
    const uint32_t m = lmax[tid];
    if (m > *(volatile uint32_t*)(gmax + tid)) atomicMax(gmax + tid, m);
  }
}

// ---------------------------------------------------------------------------------------
// accumulate
// ---------------------------------------------------------------------------------------
// record type and gradient decode per upstream-gradient dtype
template <typename GT>
struct BinRec {
  typedef uint3 type;
  __device__ static __forceinline__ type zero() { return make_uint3(0u, 0u, 0u); }
  __device__ static __forceinline__ float g0(const type& q) { return GT::to_f32((uint16_t)(q.z & 0xffffu)); }
  __device__ static __forceinline__ float g1(const type& q) { return GT::to_f32((uint16_t)(q.z >> 16)); }
  __device__ static __forceinline__ float level_max(uint32_t pattern) { return GT::to_f32((uint16_t)pattern); }
};
template <>
struct BinRec<F32> {
  typedef uint4 type;
  __device__ static __forceinline__ type zero() { return make_uint4(0u, 0u, 0u, 0u); }
  __device__ static __forceinline__ float g0(const type& q) { return __uint_as_float(q.z); }
  __device__ static __forceinline__ float g1(const type& q) { return __uint_as_float(q.w); }
  __device__ static __forceinline__ float level_max(uint32_t pattern) { return __uint_as_float(pattern); }
};

template <typename GT>
__global__ __launch_bounds__(ACC_THREADS) void hash_bwd_bin_accum_k(const typename BinRec<GT>::type* records, const uint4* tasks,
                                                                    const uint32_t* n_tasks, const uint32_t* gmax, float* dtable,
                                                                    DevGeom g, BinPlan bp, int feat, int f0) {
  typedef typename BinRec<GT>::type Rec;
  // Fixed-point sums, one plane of BIN_ROWS 64-bit cells per feature: the 64 lanes of an add go to random rows of one
  // feature, and with 8-byte cells those spread over all 64 banks (interleaved features would leave them half).
  extern __shared__ unsigned long long acc_tile[];
  if (blockIdx.x >= *n_tasks) return;
  const int tid = threadIdx.x;
  const uint4 task = tasks[blockIdx.x];
  int l = 0;
  while (l + 1 < bp.n_levels && (int)task.x >= bp.binbase[l + 1]) ++l;
  const uint32_t row0 = (task.x - (uint32_t)bp.binbase[l]) << BIN_ROWS_LOG2;
  const uint32_t left = g.rows[l] - row0;
  const uint32_t nrows = left < (uint32_t)BIN_ROWS ? left : (uint32_t)BIN_ROWS;
  // fixed-point scale 2^se of the level:  |w * g| * 2^se < 2^30
  const float gm = BinRec<GT>::level_max(gmax[l]);
  const bool nonfinite = !(gm <= 3.0e38f);
  int se = 0;
  if (!nonfinite && gm > 0.0f) {
    int ex;
    frexpf(gm, &ex);  // gm = f * 2^ex, f in [0.5, 1)
    se = 30 - ex;
    se = se > 120 ? 120 : se;
  }
  // two steps stay inside float range; the weight decode rides on the second
  const float s_lo = nonfinite ? 0.0f : ldexpf(1.0f, se / 2), s_hi = ldexpf(1.0f, se - se / 2) * (1.0f / (float)W_MAX);
  for (uint32_t i = tid; i < 2u * nrows; i += ACC_THREADS) acc_tile[(i & 1u) * BIN_ROWS + (i >> 1)] = 0ull;
  lds_barrier();
  // The task's records behind a buffer descriptor that ends with them: reads past the end return zeros (zero weights),
  // so the loop carries no bounds tests.
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<Rec*>(records + task.y), 0,
                                                                      (int)((task.z - task.y) * (uint32_t)sizeof(Rec)), 0x00020000);
  auto load_rec = [&](uint32_t at) {  // record `at` of the task
    Rec r;
    if constexpr (sizeof(Rec) == 12) {
      typedef unsigned int v3u __attribute__((ext_vector_type(3)));
      const v3u v = __builtin_amdgcn_raw_buffer_load_b96(rs, at * 12u, 0, 0);
      r.x = v[0]; r.y = v[1]; r.z = v[2];
    } else {
      typedef unsigned int v4u __attribute__((ext_vector_type(4)));
      const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rs, at * 16u, 0, 0);
      r.x = v[0]; r.y = v[1]; r.z = v[2]; r.w = v[3];
    }
    return r;
  };
  const uint32_t n_rec = task.z - task.y;
  // an odd feature count leaves the last pass with one feature: plane 1 then has no column in the table
  const bool has_pair = f0 + 1 < feat;
  // the next round's records are loaded before this round's adds; a level with an inf or a nan in its gradient only
  // marks the rows it touches (its own copy of the loop, so that the usual one has no test per record)
  auto accumulate = [&](auto nonfinite_c) {
    constexpr bool NONFINITE = decltype(nonfinite_c)::value;
    Rec q[ACC_INFLIGHT];
#pragma unroll
    for (int k = 0; k < ACC_INFLIGHT; ++k) q[k] = load_rec(k * ACC_THREADS + tid);
    for (uint32_t i0 = 0; i0 < n_rec; i0 += ACC_THREADS * ACC_INFLIGHT) {
      uint32_t slot[ACC_INFLIGHT][2];
      int32_t f[ACC_INFLIGHT][4];
#pragma unroll
      for (int k = 0; k < ACC_INFLIGHT; ++k) {
        const float g0 = BinRec<GT>::g0(q[k]) * s_lo, g1 = BinRec<GT>::g1(q[k]) * s_lo;
        const float w0 = (float)(q[k].y & W_MAX), w1 = (float)((q[k].x >> 26) << 13 | q[k].y >> W_BITS);
        slot[k][0] = q[k].x & BIN_MASK;
        slot[k][1] = (q[k].x >> BIN_ROWS_LOG2) & BIN_MASK;
        if constexpr (NONFINITE) {
          f[k][0] = w0 != 0.0f;
          f[k][2] = w1 != 0.0f;
          f[k][1] = has_pair && f[k][0];
          f[k][3] = has_pair && f[k][2];
        } else {
          f[k][0] = __float2int_rn(w0 * g0 * s_hi);
          f[k][1] = __float2int_rn(w0 * g1 * s_hi);
          f[k][2] = __float2int_rn(w1 * g0 * s_hi);
          f[k][3] = __float2int_rn(w1 * g1 * s_hi);
        }
      }
#pragma unroll
      for (int k = 0; k < ACC_INFLIGHT; ++k) q[k] = load_rec(i0 + ACC_THREADS * ACC_INFLIGHT + k * ACC_THREADS + tid);
#pragma unroll
      for (int k = 0; k < ACC_INFLIGHT; ++k)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (f[k][j]) atomicAdd(acc_tile + (uint32_t)(j & 1) * BIN_ROWS + slot[k][j >> 1], (unsigned long long)(long long)f[k][j]);
    }
  };
  // cell records (dense levels): the eight corners' rows and weights are rebuilt from the record; a corner outside this
  // bin belongs to the copy of the record in the neighbouring bin
  auto accumulate_cells = [&](auto nonfinite_c) {
    constexpr bool NONFINITE = decltype(nonfinite_c)::value;
    const uint32_t res = (uint32_t)g.res[l], r2 = res * res;
    const float s_cell = ldexpf(1.0f, se - se / 2);
    Rec q[ACC_INFLIGHT];
#pragma unroll
    for (int k = 0; k < ACC_INFLIGHT; ++k) q[k] = load_rec(k * ACC_THREADS + tid);
    for (uint32_t i0 = 0; i0 < n_rec; i0 += ACC_THREADS * ACC_INFLIGHT) {
      Rec cur[ACC_INFLIGHT];
#pragma unroll
      for (int k = 0; k < ACC_INFLIGHT; ++k) cur[k] = q[k];
#pragma unroll
      for (int k = 0; k < ACC_INFLIGHT; ++k) q[k] = load_rec(i0 + ACC_THREADS * ACC_INFLIGHT + k * ACC_THREADS + tid);
#pragma unroll
      for (int k = 0; k < ACC_INFLIGHT; ++k) {
        const bool live = (cur[k].x & 0x3fffu) != 0u;  // reads past the task's end return zero words
        const int32_t rel = (int32_t)(cur[k].x & 0x3fffu) - BIN_ROWS;
        const float fx = (float)(cur[k].x >> 14) * (1.0f / CELL_QX), fy = (float)(cur[k].y & 0xffffu) * (1.0f / CELL_QYZ),
                    fz = (float)(cur[k].y >> 16) * (1.0f / CELL_QYZ);
        const float fr[3] = {fx, fy, fz};
        float w[8];
        weights_d3(fr, w);
        const float g0 = BinRec<GT>::g0(cur[k]) * s_lo, g1 = BinRec<GT>::g1(cur[k]) * s_lo;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int32_t slot = rel + (j & 1) + ((j >> 1) & 1) * (int32_t)res + (j >> 2) * (int32_t)r2;
          if (!live || slot < 0 || slot >= BIN_ROWS) continue;
          int32_t f0v, f1v;
          if constexpr (NONFINITE) {
            f0v = w[j] != 0.0f;
            f1v = has_pair && f0v;
          } else {
            f0v = __float2int_rn(w[j] * g0 * s_cell);
            f1v = __float2int_rn(w[j] * g1 * s_cell);
          }
          if (f0v) atomicAdd(acc_tile + (uint32_t)slot, (unsigned long long)(long long)f0v);
          if (f1v) atomicAdd(acc_tile + (uint32_t)BIN_ROWS + (uint32_t)slot, (unsigned long long)(long long)f1v);
        }
      }
    }
  };
  bool cells = false;
  if constexpr (sizeof(Rec) == 12) cells = bp.cell[l] != 0;
  if (cells) {
    if (nonfinite) accumulate_cells(std::true_type{});
    else accumulate_cells(std::false_type{});
  } else if (nonfinite) accumulate(std::true_type{});
  else accumulate(std::false_type{});
  lds_barrier();
  float* dst = dtable + (g.row_offset[l] + (int64_t)row0) * feat + f0;  // features f0, f0 + 1 of the bin's rows
  const float qnan = __uint_as_float(0x7fc00000u);
  const uint32_t nvals = 2u * nrows;
  constexpr int U = 16;  // values per thread whose table reads are in flight together (a full bin in one pass)
  for (uint32_t i0 = 0; i0 < nvals; i0 += ACC_THREADS * U) {
    float x[U], old[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t i = i0 + u * ACC_THREADS + tid;
      const long long a = (i < nvals && (has_pair || !(i & 1u))) ? (long long)acc_tile[(i & 1u) * BIN_ROWS + (i >> 1)] : 0ll;
      // |a| < 2^48 is exact in double and so is the division by 2^se: one rounding, to float, at the end
      x[u] = a == 0 ? 0.0f : (float)ldexp((double)a, -se);
      if (nonfinite && a != 0) x[u] = qnan;
      old[u] = (x[u] != 0.0f && !task.w) ? dst[(i >> 1) * feat + (i & 1u)] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t i = i0 + u * ACC_THREADS + tid;
      if (x[u] != 0.0f) {
        float* cell = dst + (i >> 1) * feat + (i & 1u);
        if (task.w) unsafeAtomicAdd(cell, x[u]);
        else *cell = old[u] + x[u];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Levels of a few bins: no records
// ---------------------------------------------------------------------------------------
// When a level's table is only a few bins (the reference's default of 2^14 rows per level is two), a sorted record per
// corner pair costs more than hashing a point once per bin: a workgroup owns one bin and a slice of the points, walks
// the slice, hashes each point's corners and adds those that fall into its bin to the same 64-bit fixed-point LDS tile
// as the record kernels, then adds the tile to the table.  The upstream gradient is transposed first into level-major
// pairs, so that a bin's walk reads 4 (float32: 8) contiguous bytes per point instead of touching a whole row; the same
// pass takes the per-level maxima that set the fixed-point scales.
constexpr int DIRECT_THREADS = 1024;
constexpr int DIRECT_PREP_THREADS = 256;

// pairs[(level * np + p) * N + n] = features 2p, 2p + 1 of the level's gradient of point n (np = ceil(feat / 2); a missing
// partner is zero); gmax[level] = largest |gradient| pattern of the level over all its features
template <bool G32>
__global__ __launch_bounds__(DIRECT_PREP_THREADS) void hash_bwd_direct_prep_k(const void* dout_v, int64_t dout_stride, int64_t N,
                                                                               int levels, int feat, uint32_t* pairs, uint32_t* gmax) {
  __shared__ uint32_t lmax[NF_MAX_LEVELS];
  const int tid = threadIdx.x, lane = tid & 63;
  if (tid < NF_MAX_LEVELS) lmax[tid] = 0u;
  __syncthreads();
  const int64_t n = (int64_t)blockIdx.x * DIRECT_PREP_THREADS + tid;
  const bool valid = n < N;
  const int np = (feat + 1) / 2;
  const uint16_t* row16 = reinterpret_cast<const uint16_t*>(dout_v) + (valid ? n : 0) * dout_stride;
  const float* row32 = reinterpret_cast<const float*>(dout_v) + (valid ? n : 0) * dout_stride;
  // an even row width with 4-byte aligned rows: a pair is one dword
  const bool dword_pairs = !G32 && (feat & 1) == 0 && ((uintptr_t)dout_v & 3u) == 0 && (dout_stride & 1) == 0;
  // rows of up to sixteen levels of one pair each, 16-byte aligned: the row in four loads, level l in dword l
  const bool row_vec = !G32 && feat == 2 && levels <= 16 && (levels & 3) == 0 && ((uintptr_t)dout_v & 15u) == 0 && (dout_stride & 7) == 0;
  if (row_vec) {
    uint32_t gr[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint4 t = make_uint4(0u, 0u, 0u, 0u);
      if (valid && 4 * i < levels) t = reinterpret_cast<const uint4*>(row16)[i];
      gr[4 * i] = t.x;
      gr[4 * i + 1] = t.y;
      gr[4 * i + 2] = t.z;
      gr[4 * i + 3] = t.w;
    }
#pragma unroll
    for (int l = 0; l < 16; ++l) {
      if (l >= levels) break;
      if (valid) pairs[(int64_t)l * N + n] = gr[l];
      const uint32_t pk = gr[l] & 0x7fff7fffu;
      const uint32_t m = wave_max_u32(max(pk & 0xffffu, pk >> 16));
      if (lane == 63 && m) atomicMax(lmax + l, m);
    }
  } else
  for (int l = 0; l < levels; ++l) {
    uint32_t m = 0u;
    for (int p = 0; p < np; ++p) {
      const int e0 = l * feat + 2 * p;
      const bool two = 2 * p + 1 < feat;
      const int64_t at = ((int64_t)l * np + p) * N + n;
      if (G32) {
        uint2 pair = make_uint2(0u, 0u);
        if (valid) {
          pair.x = __float_as_uint(row32[e0]);
          if (two) pair.y = __float_as_uint(row32[e0 + 1]);
          reinterpret_cast<uint2*>(pairs)[at] = pair;
        }
        const uint32_t a0 = pair.x & 0x7fffffffu, a1 = pair.y & 0x7fffffffu;
        m = max(m, max(a0, a1));
      } else {
        uint32_t packed = 0u;
        if (valid) {
          if (dword_pairs) {
            packed = reinterpret_cast<const uint32_t*>(row16)[e0 >> 1];
          } else {
            packed = row16[e0];
            if (two) packed |= (uint32_t)row16[e0 + 1] << 16;
          }
          pairs[at] = packed;
        }
        const uint32_t pk = packed & 0x7fff7fffu;
        m = max(m, max(pk & 0xffffu, pk >> 16));
      }
    }
    m = wave_max_u32(m);
    if (lane == 63 && m) atomicMax(lmax + l, m);
  }
  __syncthreads();
  if (tid < levels) {
    const uint32_t m = lmax[tid];
    if (m > *(volatile uint32_t*)(gmax + tid)) atomicMax(gmax + tid, m);
  }
}

// blockIdx.x: a task, numbered like the bins of BinPlan; blockIdx.y: the slice of the points.  Every level here is one or
// two bins.  A level of one bin is one task whose tile holds both features of the pair; a level of two bins is two
// tasks, one per feature of the pair, whose tile holds that feature of all the level's rows: either way every corner of a
// point lands in the tile, so the walk has no test per corner and its LDS adds run with all lanes.
template <typename GT, int D>
__global__ __launch_bounds__(DIRECT_THREADS) void hash_bwd_direct_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                                     const uint32_t* pairs, int64_t N, DevGeom g, BinPlan bp,
                                                                     const int64_t* primes, float scale, const uint32_t* gmax,
                                                                     float* dtable, int feat, int p, int64_t slice_points) {
  typedef typename BinRec<GT>::type Rec;
  constexpr bool G32 = sizeof(Rec) == 16;
  extern __shared__ unsigned long long acc_tile[];  // 2 * BIN_ROWS sums
  const int tid = threadIdx.x;
  int l = 0;
  while (l + 1 < bp.n_levels && (int)blockIdx.x >= bp.binbase[l + 1]) ++l;
  const uint32_t which = blockIdx.x - (uint32_t)bp.binbase[l];
  const bool by_feature = bp.nbins[l] == 2;
  const int np = (feat + 1) / 2, f0 = 2 * p;
  const bool has_pair = f0 + 1 < feat;
  if (by_feature && which == 1u && !has_pair) return;  // an odd feature count: the last pair has one feature
  const uint32_t nrows = g.rows[l];                    // <= 2 * BIN_ROWS, and <= BIN_ROWS unless by_feature
  // fixed-point scale 2^se of the level, as in the record kernels:  |w * g| * 2^se < 2^30
  const float gm = BinRec<GT>::level_max(gmax[l]);
  const bool nonfinite = !(gm <= 3.0e38f);
  int se = 0;
  if (!nonfinite && gm > 0.0f) {
    int ex;
    frexpf(gm, &ex);
    se = 30 - ex;
    se = se > 120 ? 120 : se;
  }
  // |g| * 2^se < 2^30: the scaled gradient is a float (the two steps are exact powers of two inside float range)
  const float s_lo = nonfinite ? 0.0f : ldexpf(1.0f, se / 2), s_hi = ldexpf(1.0f, se - se / 2);
  const uint32_t ncells = by_feature ? nrows : 2u * BIN_ROWS;
  for (uint32_t i = tid; i < ncells; i += DIRECT_THREADS) acc_tile[i] = 0ull;
  lds_barrier();
  const bool hashed = l >= g.first_hash;
  const float fres = (float)g.res[l];
  const uint32_t res = (uint32_t)g.res[l], mask = g.rows[l] - 1u;
  const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], D > 2 ? (uint32_t)primes[D > 2 ? 2 : 0] : 0u};
  const uint32_t* level_pairs = pairs + (((int64_t)l * np + p) * N) * (G32 ? 2 : 1);
  const int64_t n_begin = (int64_t)blockIdx.y * slice_points;
  const int64_t n_end = n_begin + slice_points < N ? n_begin + slice_points : N;
  // One point per thread and turn: the sixteen waves of the workgroup keep enough loads in flight, and more points per
  // thread only cost registers (two: +4 %, eight: +70 %).  The loop exists in four copies, by the kind of tile and for
  // levels with an inf or a nan in their gradient (which only mark the rows they touch), so that it carries no branch.
  auto walk = [&](auto by_feature_c, auto nonfinite_c) {
    constexpr bool BY_FEATURE = decltype(by_feature_c)::value, NONFINITE = decltype(nonfinite_c)::value;
    for (int64_t n = n_begin + tid; n < n_end; n += DIRECT_THREADS) {
      float v[D > 3 ? D : 3] = {};
      Rec rec = BinRec<GT>::zero();
      load_point_d<D>(coords, cdt, csn, csd, n, scale, v);
      if constexpr (G32) {
        const uint2 t = reinterpret_cast<const uint2*>(level_pairs)[n];
        rec.z = t.x;
        rec.w = t.y;
      } else {
        rec.z = level_pairs[n];
      }
      uint32_t row[1 << D];
      float w[1 << D];
      cell_rows<D>(v, fres, hashed, res, mask, pi, primes, row, w);
      const float g0 = BinRec<GT>::g0(rec) * s_lo * s_hi, g1 = BinRec<GT>::g1(rec) * s_lo * s_hi;
      const float gs = which ? g1 : g0;
#pragma unroll
      for (int j = 0; j < (1 << D); ++j) {
        // zero contributions are rare here: the adds carry no test
        if constexpr (BY_FEATURE) {
          const int32_t fv = NONFINITE ? (int32_t)(w[j] != 0.0f) : __float2int_rn(w[j] * gs);
          atomicAdd(acc_tile + row[j], (unsigned long long)(long long)fv);
        } else {
          const int32_t f0v = NONFINITE ? (int32_t)(w[j] != 0.0f) : __float2int_rn(w[j] * g0);
          const int32_t f1v = NONFINITE ? (int32_t)(has_pair && w[j] != 0.0f) : __float2int_rn(w[j] * g1);
          atomicAdd(acc_tile + row[j], (unsigned long long)(long long)f0v);
          atomicAdd(acc_tile + (uint32_t)BIN_ROWS + row[j], (unsigned long long)(long long)f1v);
        }
      }
    }
  };
  if (by_feature) {
    if (nonfinite) walk(std::true_type{}, std::true_type{});
    else walk(std::true_type{}, std::false_type{});
  } else {
    if (nonfinite) walk(std::false_type{}, std::true_type{});
    else walk(std::false_type{}, std::false_type{});
  }
  lds_barrier();
  float* dst = dtable + g.row_offset[l] * feat + f0;
  const float qnan = __uint_as_float(0x7fc00000u);
  const uint32_t nvals = by_feature ? nrows : 2u * nrows;
  for (uint32_t i = tid; i < nvals; i += DIRECT_THREADS) {
    // by feature: value i is row i of feature `which`; else value i is feature i & 1 of row i >> 1
    const uint32_t r = by_feature ? i : i >> 1, f = by_feature ? which : (i & 1u);
    if (f && !has_pair) continue;
    const long long a = (long long)acc_tile[by_feature ? r : f * (uint32_t)BIN_ROWS + r];
    if (a == 0) continue;
    // |a| < 2^53 is exact in double and so is the division by 2^se: one rounding, to float
    const float x = nonfinite ? qnan : (float)ldexp((double)a, -se);
    if (x != 0.0f) unsafeAtomicAdd(dst + (int64_t)r * feat + f, x);
  }
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------
// Plan for levels la .. lb-1 (the kernels see them as levels 0 .. lb-la-1 of a shifted geometry).
// cells: dense 3-D levels whose eight corners span less than a bin take one record per point (16-bit gradients)
static bool bin_plan(int64_t N, const nf_hash_geom* geom, int la, int lb, BinPlan* bp, int64_t* records, uint32_t* max_tasks,
                     bool cells = false) {
  bp->n_levels = lb - la;
  int nb_total = 0;
  int64_t R = 0, R_cell = 0;
  for (int l = la; l < lb; ++l) {
    const int64_t r = geom->rows[l];
    const int64_t nb = (r + BIN_ROWS - 1) / BIN_ROWS;
    if (nb > MAX_BINS_PER_LEVEL) return false;
    bp->nbins[l - la] = (int)nb;
    bp->binbase[l - la] = nb_total;
    const int64_t res = geom->res[l];
    bp->cell[l - la] = cells && geom->dims == 3 && l < geom->first_hash_level && res * res + res + 1 < BIN_ROWS;
    // a cell level leaves at most two records per point; an x-pair level has room for every pair to be split in two
    // (normally half of it is used); more than three dimensions run as passes of the 3-D pipeline
    R += N * (bp->cell[l - la] ? 2 : geom->dims >= 3 ? 8 : 4);
    if (bp->cell[l - la]) R_cell += N * 2;
    nb_total += (int)nb;
  }
  bp->binbase[lb - la] = nb_total;
  if (nb_total > MAX_BINS_TOTAL) return false;
  if (R >= ((int64_t)1 << 32) - 4 * ACC_THREADS * ACC_INFLIGHT) return false;  // 32-bit record positions
  *records = R;
  *max_tasks = (uint32_t)(nb_total + (R - R_cell) / SPLIT_RECORDS + R_cell / (SPLIT_RECORDS / cell_task_div(N)) + 1);
  return true;
}

// The count and fill kernels keep per-bin counters of all their levels in LDS (MAX_BINS_TOTAL): tables with more bins
// go through the pipeline in groups of consecutive levels.  first[k] .. first[k+1]-1 are the levels of group k.
// (A fixed array, no heap: the entry points allocate nothing, on the host either.)
struct LevelGroups {
  int n;                             // groups
  int first[NF_MAX_LEVELS + 2];      // first[k] .. first[k + 1] - 1
  size_t size() const { return (size_t)n + 1; }
  int operator[](size_t k) const { return first[k]; }
};
static bool bin_groups(int64_t N, const nf_hash_geom* geom, LevelGroups* groups) {
  // features are taken two at a time (one pass of fill + accumulate per pair; the last feature of an odd count alone)
  if (geom->dims < 2 || geom->dims > NF_MAX_DIMS || geom->feat < 1 || N <= 0) return false;
  groups->n = 0;
  groups->first[0] = 0;
  int nb_total = 0;
  for (int l = 0; l < geom->levels; ++l) {
    const int64_t nb = (geom->rows[l] + BIN_ROWS - 1) / BIN_ROWS;
    if (nb > MAX_BINS_PER_LEVEL) return false;
    if (nb_total + nb > MAX_BINS_TOTAL) {
      groups->first[++groups->n] = l;
      nb_total = 0;
    }
    nb_total += (int)nb;
  }
  groups->first[++groups->n] = geom->levels;
  for (int k = 0; k < groups->n; ++k) {
    BinPlan bp;
    int64_t R;
    uint32_t mt;
    if (!bin_plan(N, geom, groups->first[k], groups->first[k + 1], &bp, &R, &mt)) return false;
  }
  return true;
}

static int64_t wg_count_words(int64_t N, int NB) { return (((N + FILL_POINTS - 1) / FILL_POINTS) * NB + 3) & ~(int64_t)3; }

static int64_t bin_ws(void* workspace, const BinPlan& bp, int64_t N, int64_t R, int rec_words, uint32_t max_tasks, BinWs* ws) {
  uint32_t* p = (uint32_t*)workspace;
  const int NB = bp.binbase[bp.n_levels];
  const int NBp = (NB + 3) & ~3;
  int64_t o = 0;
  ws->hist = p + o; o += NBp;
  ws->gmax = p + o; o += 32;
  ws->cursor = p + o; o += NBp;
  ws->n_tasks = p + o; o += 4;
  ws->tasks = reinterpret_cast<uint4*>(p + o); o += 4 * (int64_t)max_tasks;
  ws->wg_counts = p + o; o += wg_count_words(N, NB);
  o = (o + 3) & ~(int64_t)3;  // 16-byte records start on a 16-byte boundary
  ws->records = p + o; o += (int64_t)rec_words * R;
  ws->max_tasks = max_tasks;
  return o * 4;
}

// Batches above this many points go through the pipeline in pieces of this size, one after the other on the stream:
// the scratch stays at ~3 GiB (4 GiB with a float32 upstream gradient) whatever the batch, and record positions stay
// inside 32 bits.  The gradient table accumulates across the pieces.  (Pieces of 2^20 points would halve the scratch
// and cost 2.5 % of a 2^21-point training step: every piece pays the fixed part of the pipeline again.)
constexpr int64_t BIN_CHUNK_POINTS = (int64_t)1 << 21;

// The walk without records hashes every point once per task of a level (two for a level of two bins); the records pay a
// count, a fill and an accumulate pass per level whatever its size.  With every level at most two bins (2^14 rows, the
// reference's default table size) the walk is the faster one; four bins would already cost it more hashing than the
// records' passes take.
constexpr int DIRECT_MAX_BINS_PER_LEVEL = 2;
constexpr int DIRECT_MAX_DIMS = 4;  // the walk is built for 1 to 4 dimensions (the sorted records for 2 and 3)
constexpr int64_t DIRECT_MIN_POINTS = 4096;  // below: one launch of scattered atomics is as quick
static bool direct_ok(int64_t n_points, const nf_hash_geom* geom, int flags) {
  if ((flags & NF_HASH_BWD_RECORDS) || n_points < DIRECT_MIN_POINTS) return false;
  if (geom->dims < 1 || geom->dims > DIRECT_MAX_DIMS) return false;
  for (int l = 0; l < geom->levels; ++l)
    if (geom->rows[l] > (int64_t)DIRECT_MAX_BINS_PER_LEVEL * BIN_ROWS) return false;
  return true;
}
bool bwd_direct_applies(int64_t n_points, const nf_hash_geom* geom, int flags) {
  return direct_ok(n_points < BIN_CHUNK_POINTS ? n_points : BIN_CHUNK_POINTS, geom, flags);
}
// gmax[32] (padded to 256 bytes) | pairs[levels][ceil(feat / 2)][n_points] of 4 (float32 gradient: 8) bytes
static int64_t direct_workspace_bytes(int64_t n_points, const nf_hash_geom* geom, int dout_dtype) {
  return 256 + (int64_t)geom->levels * ((geom->feat + 1) / 2) * n_points * (dout_dtype == NF_F32 ? 8 : 4);
}

int64_t bwd_bin_workspace_bytes(int64_t n_points, const nf_hash_geom* geom, int dout_dtype, int flags) {
  if (n_points > BIN_CHUNK_POINTS) n_points = BIN_CHUNK_POINTS;
  if (direct_ok(n_points, geom, flags)) return direct_workspace_bytes(n_points, geom, dout_dtype);
  LevelGroups first;
  if (!bin_groups(n_points, geom, &first)) return 0;
  int64_t bytes = 0;
  for (size_t k = 0; k + 1 < first.size(); ++k) {
    BinPlan bp;
    int64_t R;
    uint32_t max_tasks;
    bin_plan(n_points, geom, first[k], first[k + 1], &bp, &R, &max_tasks, dout_dtype != NF_F32);
    BinWs ws;
    const int64_t b = bin_ws(nullptr, bp, n_points, R, dout_dtype == NF_F32 ? 4 : 3, max_tasks, &ws);
    if (b > bytes) bytes = b;
  }
  return bytes;
}

static int launch_bwd_bin_group(const void* coords, int cdt, int64_t csn, int64_t csd, const void* dout, int ddt, int64_t dout_stride,
                                float* dtable, int64_t N, const nf_hash_geom* geom, const DevGeom& g, const BinPlan& bp, int64_t R,
                                uint32_t max_tasks, const int64_t* primes, float scale, void* workspace, hipStream_t s);

static int launch_bwd_bin_piece(const void* coords, int cdt, int64_t csn, int64_t csd, const void* dout, int ddt, int64_t dout_stride,
                                float* dtable, int64_t N, const nf_hash_geom* geom, const DevGeom& g, const int64_t* primes, float scale,
                                void* workspace, hipStream_t s);

static int launch_bwd_direct(const void* coords, int cdt, int64_t csn, int64_t csd, const void* dout, int ddt, int64_t dout_stride,
                             float* dtable, int64_t N, const nf_hash_geom* geom, const DevGeom& g, const int64_t* primes, float scale,
                             void* workspace, hipStream_t s);

int launch_bwd_bin(const void* coords, int cdt, int64_t csn, int64_t csd, const void* dout, int ddt, int64_t dout_stride,
                   float* dtable, int64_t N, const nf_hash_geom* geom, const DevGeom& g, const int64_t* primes, float scale,
                   void* workspace, int flags, hipStream_t s) {
  // the choice is made once, on the size the workspace was asked for: every piece then fits it
  const bool direct = direct_ok(N < BIN_CHUNK_POINTS ? N : BIN_CHUNK_POINTS, geom, flags);
  for (int64_t n0 = 0; n0 < N; n0 += BIN_CHUNK_POINTS) {
    const int64_t n = N - n0 < BIN_CHUNK_POINTS ? N - n0 : BIN_CHUNK_POINTS;
    const char* c = (const char*)coords + n0 * csn * dtype_size(cdt);
    const char* d = (const char*)dout + n0 * dout_stride * dtype_size(ddt);
    const int rc = direct ? launch_bwd_direct(c, cdt, csn, csd, d, ddt, dout_stride, dtable, n, geom, g, primes, scale, workspace, s)
                          : launch_bwd_bin_piece(c, cdt, csn, csd, d, ddt, dout_stride, dtable, n, geom, g, primes, scale, workspace, s);
    if (rc) return rc;
  }
  return 0;
}

static int direct_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) cus = p.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

static int launch_bwd_direct(const void* coords, int cdt, int64_t csn, int64_t csd, const void* dout, int ddt, int64_t dout_stride,
                             float* dtable, int64_t N, const nf_hash_geom* geom, const DevGeom& g, const int64_t* primes, float scale,
                             void* workspace, hipStream_t s) {
  NF_REQUIRE(((uintptr_t)workspace & 15u) == 0, NF_EALIGN, "workspace must be 16-byte aligned");
  BinPlan bp;
  int64_t R;
  uint32_t max_tasks;
  NF_REQUIRE(bin_plan(N, geom, 0, geom->levels, &bp, &R, &max_tasks, false), NF_EUNSUPPORTED,
             "backward without records does not cover this geometry");
  const int NB = bp.binbase[bp.n_levels];
  uint32_t* gmax = reinterpret_cast<uint32_t*>(workspace);
  uint32_t* pairs = gmax + 64;
  const bool g32 = ddt == NF_F32;
  hipLaunchKernelGGL(hash_bwd_bin_zero_k, dim3(1), dim3(64), 0, s, gmax, 32);
  if (int rc = check_launch("hash_bwd_bin_zero")) return rc;
  const unsigned prep_blocks = (unsigned)((N + DIRECT_PREP_THREADS - 1) / DIRECT_PREP_THREADS);
  if (g32)
    hipLaunchKernelGGL(hash_bwd_direct_prep_k<true>, dim3(prep_blocks), dim3(DIRECT_PREP_THREADS), 0, s, dout, dout_stride, N,
                       g.levels, g.feat, pairs, gmax);
  else
    hipLaunchKernelGGL(hash_bwd_direct_prep_k<false>, dim3(prep_blocks), dim3(DIRECT_PREP_THREADS), 0, s, dout, dout_stride, N,
                       g.levels, g.feat, pairs, gmax);
  if (int rc = check_launch("hash_bwd_direct_prep")) return rc;
  // at most two workgroups per compute unit in all, so that they run as two full rounds (one fits at a time: the tile is
  // 128 KiB of LDS; four rounds: +3 %, eight: +11 %), in slices of whole turns of the point loop and of at least 4096 points
  const int64_t round = (int64_t)DIRECT_THREADS;
  int64_t slices = (int64_t)2 * direct_cus() / NB;
  if (slices < 1) slices = 1;
  int64_t slice_points = (N + slices - 1) / slices;
  if (slice_points < 4096) slice_points = 4096;
  slice_points = (slice_points + round - 1) / round * round;
  slices = (N + slice_points - 1) / slice_points;
  const size_t lds = (size_t)2 * BIN_ROWS * sizeof(unsigned long long);
  auto pick = [&](auto d_c) -> const void* {
    constexpr int DD = decltype(d_c)::value;
    return ddt == NF_F32 ? (const void*)hash_bwd_direct_k<F32, DD> : ddt == NF_BF16 ? (const void*)hash_bwd_direct_k<BF16, DD> : (const void*)hash_bwd_direct_k<F16, DD>;
  };
  const void* kern = g.dims == 3   ? pick(std::integral_constant<int, 3>{})
                     : g.dims == 2 ? pick(std::integral_constant<int, 2>{})
                     : g.dims == 1 ? pick(std::integral_constant<int, 1>{})
                                   : pick(std::integral_constant<int, 4>{});
  hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  const uint32_t* cpairs = pairs;
  const uint32_t* cgmax = gmax;
  const int feat = geom->feat;
  for (int p = 0; p < (feat + 1) / 2; ++p) {
    void* args[] = {(void*)&coords, (void*)&cdt, (void*)&csn, (void*)&csd, (void*)&cpairs, (void*)&N, (void*)&g, (void*)&bp,
                    (void*)&primes, (void*)&scale, (void*)&cgmax, (void*)&dtable, (void*)&feat, (void*)&p, (void*)&slice_points};
    e = hipLaunchKernel(kern, dim3((unsigned)NB, (unsigned)slices), dim3(DIRECT_THREADS), args, lds, s);
    if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(hash_bwd_direct): %s", hipGetErrorString(e));
    if (int rc = check_launch("hash_bwd_direct")) return rc;
  }
  return 0;
}

static int launch_bwd_bin_piece(const void* coords, int cdt, int64_t csn, int64_t csd, const void* dout, int ddt, int64_t dout_stride,
                                float* dtable, int64_t N, const nf_hash_geom* geom, const DevGeom& g, const int64_t* primes, float scale,
                                void* workspace, hipStream_t s) {
  LevelGroups first;
  NF_REQUIRE(bin_groups(N, geom, &first), NF_EUNSUPPORTED, "binned backward does not cover this geometry");
  NF_REQUIRE(((uintptr_t)workspace & 15u) == 0, NF_EALIGN, "workspace must be 16-byte aligned");
  for (size_t k = 0; k + 1 < first.size(); ++k) {
    const int la = first[k], lb = first[k + 1];
    BinPlan bp;
    int64_t R;
    uint32_t max_tasks;
    bin_plan(N, geom, la, lb, &bp, &R, &max_tasks, ddt != NF_F32);
    // the group's levels as levels 0 .. of a geometry of their own; their gradient columns start at la * feat
    DevGeom gg = g;
    gg.levels = lb - la;
    gg.first_hash = g.first_hash - la;
    for (int l = la; l < lb; ++l) {
      gg.res[l - la] = g.res[l];
      gg.rows[l - la] = g.rows[l];
      gg.row_offset[l - la] = g.row_offset[l];
    }
    const char* dcol = (const char*)dout + (size_t)la * geom->feat * (ddt == NF_F32 ? 4 : 2);
    if (int rc = launch_bwd_bin_group(coords, cdt, csn, csd, dcol, ddt, dout_stride, dtable, N, geom, gg, bp, R, max_tasks, primes,
                                      scale, workspace, s))
      return rc;
  }
  return 0;
}

static int launch_bwd_bin_group(const void* coords, int cdt, int64_t csn, int64_t csd, const void* dout, int ddt, int64_t dout_stride,
                                float* dtable, int64_t N, const nf_hash_geom* geom, const DevGeom& g, const BinPlan& bp, int64_t R,
                                uint32_t max_tasks, const int64_t* primes, float scale, void* workspace, hipStream_t s) {
  const bool g32 = ddt == NF_F32;
  BinWs ws;
  bin_ws(workspace, bp, N, R, g32 ? 4 : 3, max_tasks, &ws);
  const int NB = bp.binbase[bp.n_levels];
  const int NBp = (NB + 3) & ~3;
  const unsigned blocks = (unsigned)((N + FILL_POINTS - 1) / FILL_POINTS);

  // more than three dimensions: the whole pipeline once per corner of the extra coordinates (`hi`), see ExtraDims
  const int passes = g.dims > 3 ? 1 << (g.dims - 3) : 1;
  for (int hi = 0; hi < passes; ++hi) {
  hipLaunchKernelGGL(hash_bwd_bin_zero_k, dim3((unsigned)((NBp + 32 + 255) / 256)), dim3(256), 0, s, ws.hist, NBp + 32);
  if (int rc = check_launch("hash_bwd_bin_zero")) return rc;
  if (g.dims == 6)
    hipLaunchKernelGGL((hash_bwd_bin_count_k<3, 3>), dim3(blocks), dim3(FILL_POINTS), (size_t)NB * 4, s, coords, cdt, csn, csd, N, g, bp,
                       primes, scale, ws.hist, ws.wg_counts, hi);
  else if (g.dims == 5)
    hipLaunchKernelGGL((hash_bwd_bin_count_k<3, 2>), dim3(blocks), dim3(FILL_POINTS), (size_t)NB * 4, s, coords, cdt, csn, csd, N, g, bp,
                       primes, scale, ws.hist, ws.wg_counts, hi);
  else if (g.dims == 4)
    hipLaunchKernelGGL((hash_bwd_bin_count_k<3, 1>), dim3(blocks), dim3(FILL_POINTS), (size_t)NB * 4, s, coords, cdt, csn, csd, N, g, bp,
                       primes, scale, ws.hist, ws.wg_counts, hi);
  else if (g.dims == 3)
    hipLaunchKernelGGL(hash_bwd_bin_count_k<3>, dim3(blocks), dim3(FILL_POINTS), (size_t)NB * 4, s, coords, cdt, csn, csd, N, g, bp,
                       primes, scale, ws.hist, ws.wg_counts, hi);
  else
    hipLaunchKernelGGL(hash_bwd_bin_count_k<2>, dim3(blocks), dim3(FILL_POINTS), (size_t)NB * 4, s, coords, cdt, csn, csd, N, g, bp,
                       primes, scale, ws.hist, ws.wg_counts, hi);
  if (int rc = check_launch("hash_bwd_bin_count")) return rc;
  hipLaunchKernelGGL(hash_bwd_bin_offsets_k, dim3(1), dim3(1024), 0, s, (const uint32_t*)ws.hist, ws.cursor, ws.n_tasks,
                     ws.tasks, NB, max_tasks, bp, cell_task_div(N));
  if (int rc = check_launch("hash_bwd_bin_offsets")) return rc;
  const int feat = geom->feat;
  for (int f0 = 0; f0 < feat; f0 += 2) {
    if (f0 > 0) {
      // the next pair of features: same bins and tasks; fresh level maxima and bin cursors
      hipLaunchKernelGGL(hash_bwd_bin_zero_k, dim3(1), dim3(256), 0, s, ws.gmax, 32);
      if (int rc = check_launch("hash_bwd_bin_zero")) return rc;
      hipLaunchKernelGGL(hash_bwd_bin_offsets_k, dim3(1), dim3(1024), 0, s, (const uint32_t*)ws.hist, ws.cursor, ws.n_tasks,
                         ws.tasks, NB, max_tasks, bp, cell_task_div(N));
      if (int rc = check_launch("hash_bwd_bin_offsets")) return rc;
    }
  {
    const size_t lds = (size_t)FILL_RECORDS * sizeof(uint4) + (g32 ? (size_t)FILL_POINTS * sizeof(uint2) : 0) +
                       ((size_t)2 * NB + 2 * NF_MAX_LEVELS) * 4;
    const void* kern = g.dims == 6   ? (g32 ? (const void*)hash_bwd_bin_fill_k<true, 3, 3> : (const void*)hash_bwd_bin_fill_k<false, 3, 3>)
                       : g.dims == 5 ? (g32 ? (const void*)hash_bwd_bin_fill_k<true, 3, 2> : (const void*)hash_bwd_bin_fill_k<false, 3, 2>)
                       : g.dims == 4 ? (g32 ? (const void*)hash_bwd_bin_fill_k<true, 3, 1> : (const void*)hash_bwd_bin_fill_k<false, 3, 1>)
                       : g.dims == 3 ? (g32 ? (const void*)hash_bwd_bin_fill_k<true, 3> : (const void*)hash_bwd_bin_fill_k<false, 3>)
                                     : (g32 ? (const void*)hash_bwd_bin_fill_k<true, 2> : (const void*)hash_bwd_bin_fill_k<false, 2>);
    hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    const uint32_t* wc = ws.wg_counts;
    void* args[] = {(void*)&coords, (void*)&cdt,   (void*)&csn,    (void*)&csd,   (void*)&dout, (void*)&dout_stride, (void*)&N, (void*)&g,
                    (void*)&bp,     (void*)&primes, (void*)&scale, (void*)&wc,    (void*)&ws.cursor, (void*)&ws.gmax, (void*)&ws.records,
                    (void*)&feat,   (void*)&f0,     (void*)&hi};
    e = hipLaunchKernel(kern, dim3(blocks), dim3(FILL_POINTS), args, lds, s);
    if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(hash_bwd_bin_fill): %s", hipGetErrorString(e));
    if (int rc = check_launch("hash_bwd_bin_fill")) return rc;
  }
  {
    const size_t lds = (size_t)BIN_ROWS * 2 * sizeof(unsigned long long);
    const void* kern = ddt == NF_F16    ? (const void*)hash_bwd_bin_accum_k<F16>
                       : ddt == NF_BF16 ? (const void*)hash_bwd_bin_accum_k<BF16>
                                        : (const void*)hash_bwd_bin_accum_k<F32>;
    hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    const uint32_t* rc_ = ws.records;
    const uint4* tk = ws.tasks;
    const uint32_t* nt = ws.n_tasks;
    const uint32_t* gm = ws.gmax;
    void* args[] = {(void*)&rc_, (void*)&tk, (void*)&nt, (void*)&gm, (void*)&dtable, (void*)&g, (void*)&bp, (void*)&feat, (void*)&f0};
    e = hipLaunchKernel(kern, dim3(max_tasks), dim3(ACC_THREADS), args, lds, s);
    if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(hash_bwd_bin_accum): %s", hipGetErrorString(e));
    if (int rc = check_launch("hash_bwd_bin_accum")) return rc;
  }
  }
  }
  return 0;
}

}  // namespace nf
