// Hash-encoding backward without scattered global atomics (D = 3, F = 2, 16-bit upstream gradient).
//
// Measured on MI355X: a global float atomic costs one request slot per 64-byte segment at about
// 21 G requests/s for the whole chip, whatever the table size or scope, so 2^20 points x 16 levels
// x 8 corners x 2 features scattered one by one take ~13 ms.  LDS integer atomics and LDS
// compare-and-swap are two orders of magnitude faster, so the gradient of every level is
// accumulated in LDS instead:
//
//   * A level's gradient table is cut into tiles of TILE_ROWS rows (128 KiB of float2).  One
//     workgroup owns one (level, tile, slice of the points), accumulates into its LDS tile with a
//     64-bit compare-and-swap add (both features of a row at once), and finally adds the tile to
//     the global table with coalesced atomics (16 floats per request).
//   * A workgroup must only look at the points that touch its tile.  A first kernel (plan) writes,
//     per (level, tile), one bit per point -- "some corner of this point falls into this tile" --
//     so an owner reads N/8 bytes of bit-plane instead of all N points, expands the set bits into a
//     per-wave queue of point indices and processes them 64 at a time with all lanes busy.
//   * Levels that fit one tile need no bit-plane: every point hits.
//
// Arithmetic (cell, corner rows, weights) is the forward's, see hash_encoding.hip.
#include "hash_common.h"

namespace nf {

constexpr int TILE_ROWS_LOG2 = 14;
constexpr int TILE_ROWS = 1 << TILE_ROWS_LOG2;  // rows per LDS tile (float2 each: 128 KiB)
constexpr int SCAN_THREADS = 1024;
constexpr int SCAN_WAVES = SCAN_THREADS / 64;
constexpr int QUEUE_CAP = 128;     // per-wave queue entries (< 64 pending + <= 64 appended per round)
constexpr int PLAN_POINTS = 1024;  // points per plan workgroup == 32 bit-plane words
constexpr int64_t HITS_PER_TASK_HASHED = 65536;  // (point, corner pair) hits per workgroup, hashed levels
constexpr int64_t HITS_PER_TASK_DENSE = 8192;    // points per workgroup where all 8 corners of a point land in the tile

struct ScanPlan {
  int n_levels;
  int planes_pad;                 // planes rounded up to an odd number (LDS bank spread in the plan kernel)
  int64_t words;                  // 32-bit words per bit-plane
  int tiles[NF_MAX_LEVELS];       // tiles of the level
  int plane0[NF_MAX_LEVELS];      // first bit-plane of the level, -1: single tile, no planes
  int slices[NF_MAX_LEVELS];      // point slices per tile
  // Tasks are ordered slice-major so that the workgroups running at the same time walk the same part of the
  // point array (their coordinate / gradient reads then meet in L2).  Levels have different slice counts, so the
  // order is cut into segments: within segment k every slice index s in [seg_s0[k], seg_s0[k+1]) contributes one
  // task per tile of every level with slices[l] > s, levels in ascending order.
  int n_segs;
  int seg_s0[NF_MAX_LEVELS + 2];    // first slice index of the segment
  int seg_task0[NF_MAX_LEVELS + 2]; // first task of the segment
  int seg_width[NF_MAX_LEVELS + 1]; // tasks per slice index inside the segment
  int n_tasks;
  int xfree[NF_MAX_LEVELS];       // hashed level whose tile id does not depend on the x corner (res + 1 <= TILE_ROWS)
};

struct Located {
  uint32_t c[3];
  float fr[3];
};

__device__ __forceinline__ Located locate3(const void* coords, int cdt, int64_t csn, int64_t csd, int64_t n, float scale,
                                           float fres) {
  Located r;
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    float v = load_as_f32(coords, n * csn + d * csd, cdt);
    if (scale != 1.0f) v = v / scale;
    const float pos = v * fres;
    const float fl = floorf(pos);
    r.c[d] = cell_index(fl, fres);
    r.fr[d] = pos - fl;
  }
  return r;
}

// ---------------------------------------------------------------------------------------
// Plan: one bit per (level, tile, point)
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(PLAN_POINTS) void hash_bwd_plan_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                               const uint16_t* dout, int64_t dout_stride, uint32_t* planes,
                                                               uint32_t* gT, int64_t N, DevGeom g, ScanPlan sp,
                                                               const int64_t* primes, float scale) {
  extern __shared__ uint32_t bm[];  // [32 words][planes_pad]
  const int tid = threadIdx.x;
  const int P = sp.planes_pad;
  for (int i = tid; i < 32 * P; i += PLAN_POINTS) bm[i] = 0u;
  __syncthreads();
  const int64_t n = (int64_t)blockIdx.x * PLAN_POINTS + tid;
  if (n < N) {
    const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], (uint32_t)primes[2]};
    uint32_t* row = bm + (tid >> 5) * P;
    const uint32_t bit = 1u << (tid & 31);
    // this point's gradient row, read once (up to 16 levels live in registers)
    const uint32_t* grow = reinterpret_cast<const uint32_t*>(dout + n * dout_stride);
    uint32_t gr[16];
    const bool row_vec = sp.n_levels <= 16 && (sp.n_levels & 3) == 0 && ((uintptr_t)grow & 15u) == 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (row_vec && 4 * i < sp.n_levels) v = reinterpret_cast<const uint4*>(grow)[i];
      gr[4 * i] = v.x;
      gr[4 * i + 1] = v.y;
      gr[4 * i + 2] = v.z;
      gr[4 * i + 3] = v.w;
    }
    for (int l = 0; l < sp.n_levels; ++l) {
      // the level's packed upstream gradient, transposed to gT[level][point] for the scan's reads
      uint32_t packed;
      if (row_vec) {
        packed = gr[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) packed = (l == i) ? gr[i] : packed;
      } else {
        packed = grow[l];
      }
      gT[(int64_t)l * sp.words * 32 + n] = packed;
      if (sp.plane0[l] < 0 || (packed & 0x7fff7fffu) == 0u) continue;  // no planes, or nothing to scatter
      const Located q = locate3(coords, cdt, csn, csd, n, scale, (float)g.res[l]);
      uint32_t* lrow = row + sp.plane0[l];
      if (l >= g.first_hash) {
        const uint32_t mask = g.rows[l] - 1;
        const uint32_t y0 = q.c[1] * pi[1], y1 = y0 + pi[1];
        const uint32_t z0 = q.c[2] * pi[2], z1 = z0 + pi[2];
        const uint32_t x0 = q.c[0] * pi[0], x1 = x0 + pi[0];
        if (sp.xfree[l]) {
          atomicOr(lrow + (((x0 ^ y0 ^ z0) & mask) >> TILE_ROWS_LOG2), bit);
          atomicOr(lrow + (((x0 ^ y1 ^ z0) & mask) >> TILE_ROWS_LOG2), bit);
          atomicOr(lrow + (((x0 ^ y0 ^ z1) & mask) >> TILE_ROWS_LOG2), bit);
          atomicOr(lrow + (((x0 ^ y1 ^ z1) & mask) >> TILE_ROWS_LOG2), bit);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const uint32_t h = ((j & 1 ? x1 : x0) ^ (j & 2 ? y1 : y0) ^ (j & 4 ? z1 : z0)) & mask;
            atomicOr(lrow + (h >> TILE_ROWS_LOG2), bit);
          }
        }
      } else {
        // dense: the 8 corner rows span [b, b + res^2 + res + 1]
        const uint32_t res = (uint32_t)g.res[l], r2 = res * res;
        const uint32_t b = q.c[0] + q.c[1] * res + q.c[2] * r2;
        const uint32_t t_lo = b >> TILE_ROWS_LOG2, t_hi = (b + r2 + res + 1) >> TILE_ROWS_LOG2;
        for (uint32_t t = t_lo; t <= t_hi && (int)t < sp.tiles[l]; ++t) atomicOr(lrow + t, bit);
      }
    }
  }
  __syncthreads();
  // planes[plane][word]: every plane gets this workgroup's 32 consecutive words
  int n_planes = 0;
  for (int l = 0; l < sp.n_levels; ++l)
    if (sp.plane0[l] >= 0) n_planes = sp.plane0[l] + sp.tiles[l];
  for (int i = tid; i < n_planes * 32; i += PLAN_POINTS) {
    const int plane = i >> 5, w = i & 31;
    planes[(int64_t)plane * sp.words + (int64_t)blockIdx.x * 32 + w] = bm[w * P + plane];
  }
}

// ---------------------------------------------------------------------------------------
// Scan: one workgroup per (level, tile, slice)
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ void lds_add2(float2* slot, float v0, float v1) {
  unsigned long long* p = reinterpret_cast<unsigned long long*>(slot);
  unsigned long long old = *p, assumed;
  do {
    assumed = old;
    const float a = __uint_as_float((uint32_t)assumed) + v0;
    const float b = __uint_as_float((uint32_t)(assumed >> 32)) + v1;
    old = atomicCAS(p, assumed, (unsigned long long)__float_as_uint(a) | ((unsigned long long)__float_as_uint(b) << 32));
  } while (old != assumed);
}

// What a lane needs of one queued point: raw coordinates and the level's packed upstream gradient.
struct PointData {
  float x[3];
  uint32_t packed;
};

// FAST: float32 coordinates stored [N][3] contiguously, scale 1, 3*N below 2^31.
// gl: this level's row of the transposed gradient (one dword per point).
template <bool FAST>
__device__ __forceinline__ PointData fetch_point(uint32_t n, const void* coords, int cdt, int64_t csn, int64_t csd,
                                                 const uint32_t* gl) {
  PointData p;
  if (FAST) {
    const float* c = reinterpret_cast<const float*>(coords) + n * 3u;
    p.x[0] = c[0];
    p.x[1] = c[1];
    p.x[2] = c[2];
  } else {
#pragma unroll
    for (int d = 0; d < 3; ++d) p.x[d] = load_as_f32(coords, (int64_t)n * csn + d * csd, cdt);
  }
  p.packed = gl[n];
  return p;
}

__device__ __forceinline__ unsigned long long add2_bits(unsigned long long old, float v0, float v1) {
  const float a = __uint_as_float((uint32_t)old) + v0;
  const float b = __uint_as_float((uint32_t)(old >> 32)) + v1;
  return (unsigned long long)__float_as_uint(a) | ((unsigned long long)__float_as_uint(b) << 32);
}

// K independent float2 += (v0, v1) on LDS slots by 64-bit compare-and-swap, all K in flight at once.
template <int K>
__device__ __forceinline__ void lds_add2_multi(float2* tile, const uint32_t (&slot)[K], const bool (&on)[K], const float (&v0)[K],
                                               const float (&v1)[K]) {
  unsigned long long old[K];
  bool todo[K];
  bool any = false;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    todo[k] = on[k];
    any = any || on[k];
    if (on[k]) old[k] = *reinterpret_cast<unsigned long long*>(tile + slot[k]);
  }
  while (any) {
    unsigned long long got[K];
#pragma unroll
    for (int k = 0; k < K; ++k)
      if (todo[k]) got[k] = atomicCAS(reinterpret_cast<unsigned long long*>(tile + slot[k]), old[k], add2_bits(old[k], v0[k], v1[k]));
    any = false;
#pragma unroll
    for (int k = 0; k < K; ++k)
      if (todo[k]) {
        todo[k] = got[k] != old[k];
        old[k] = got[k];
        any = any || todo[k];
      }
  }
}

template <typename GT>
__device__ __forceinline__ void scatter_point(float2* tile, uint32_t tile_id, const PointData& p, int l, bool hashed, bool xfree,
                                              const DevGeom& g, const uint32_t (&pi)[3], float scale) {
  if ((p.packed & 0x7fff7fffu) == 0u) return;  // zero upstream gradient for both features
  const float g0 = GT::to_f32((uint16_t)(p.packed & 0xffffu));
  const float g1 = GT::to_f32((uint16_t)(p.packed >> 16));
  const uint32_t res = (uint32_t)g.res[l];
  const float fres = (float)g.res[l];
  Located q;
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    const float v = scale != 1.0f ? p.x[d] / scale : p.x[d];
    const float pos = v * fres;
    const float fl = floorf(pos);
    q.c[d] = cell_index(fl, fres);
    q.fr[d] = pos - fl;
  }
  if (hashed && xfree) {
    // The tile id of a corner does not depend on its x offset: test the four (y, z) pairs, then handle
    // the matching pairs one per round (a lane usually has exactly one), the x pair of each in flight together.
    const uint32_t mask = g.rows[l] - 1;
    const uint32_t y0 = q.c[1] * pi[1], y1 = y0 + pi[1];
    const uint32_t z0 = q.c[2] * pi[2], z1 = z0 + pi[2];
    const uint32_t m0 = (y0 ^ z0) & mask, m1 = (y1 ^ z0) & mask, m2 = (y0 ^ z1) & mask, m3 = (y1 ^ z1) & mask;
    uint32_t match = ((m0 >> TILE_ROWS_LOG2) == tile_id ? 1u : 0u) | ((m1 >> TILE_ROWS_LOG2) == tile_id ? 2u : 0u) |
                     ((m2 >> TILE_ROWS_LOG2) == tile_id ? 4u : 0u) | ((m3 >> TILE_ROWS_LOG2) == tile_id ? 8u : 0u);
    const float fx = q.fr[0], gx = 1.0f - fx;
    const uint32_t x0 = q.c[0] * pi[0], x1 = x0 + pi[0];
    while (match != 0u) {
      const uint32_t j = (uint32_t)__ffs((int)match) - 1u;
      match &= match - 1u;
      const uint32_t m = j == 0u ? m0 : (j == 1u ? m1 : (j == 2u ? m2 : m3));
      const float wy = (j & 1u) ? q.fr[1] : 1.0f - q.fr[1];
      const float wz = (j & 2u) ? q.fr[2] : 1.0f - q.fr[2];
      const float w0 = (gx * wy) * wz, w1 = (fx * wy) * wz;
      const uint32_t slot[2] = {(x0 ^ m) & (TILE_ROWS - 1), (x1 ^ m) & (TILE_ROWS - 1)};
      const bool on[2] = {true, true};
      const float v0[2] = {w0 * g0, w1 * g0};
      const float v1[2] = {w0 * g1, w1 * g1};
      lds_add2_multi<2>(tile, slot, on, v0, v1);
    }
  } else {
    float w[8];
    weights_d3(q.fr, w);
    const Corner8 r = rows_d3(q.c, hashed, res, g.rows[l] - 1, pi);
    uint32_t slot[8];
    bool on[8];
    float v0[8], v1[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      on[j] = (r.row[j] >> TILE_ROWS_LOG2) == tile_id;
      slot[j] = r.row[j] & (TILE_ROWS - 1);
      v0[j] = w[j] * g0;
      v1[j] = w[j] * g1;
    }
    lds_add2_multi<8>(tile, slot, on, v0, v1);
  }
}

template <typename GT, bool FAST>
__global__ __launch_bounds__(SCAN_THREADS) void hash_bwd_scan_k(const void* coords, int cdt, int64_t csn, int64_t csd,
                                                                const uint32_t* gT, float* dtable, const uint32_t* planes,
                                                                int64_t N, DevGeom g, ScanPlan sp, const int64_t* primes,
                                                                float scale) {
  extern __shared__ __align__(16) unsigned char smem[];
  float2* tile = reinterpret_cast<float2*>(smem);
  uint32_t* queues = reinterpret_cast<uint32_t*>(smem + (size_t)TILE_ROWS * sizeof(float2));
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // ---- which (level, tile, slice) is this workgroup
  int seg = 0;
  while (seg + 1 < sp.n_segs && (int)blockIdx.x >= sp.seg_task0[seg + 1]) ++seg;
  const int in_seg = (int)blockIdx.x - sp.seg_task0[seg];
  const int slice = sp.seg_s0[seg] + in_seg / sp.seg_width[seg];
  int rest = in_seg % sp.seg_width[seg];
  int l = 0;
  for (; l < sp.n_levels; ++l) {
    if (sp.slices[l] <= slice) continue;
    if (rest < sp.tiles[l]) break;
    rest -= sp.tiles[l];
  }
  const int n_slices = sp.slices[l];
  const uint32_t tile_id = (uint32_t)rest;
  const uint32_t* gl = gT + (int64_t)l * sp.words * 32;
  const bool hashed = l >= g.first_hash;
  const bool xfree = sp.xfree[l] != 0;
  const uint32_t pi[3] = {(uint32_t)primes[0], (uint32_t)primes[1], (uint32_t)primes[2]};

  const int64_t row0 = (int64_t)tile_id * TILE_ROWS;
  const int rows_here = (int)((int64_t)g.rows[l] - row0 < TILE_ROWS ? (int64_t)g.rows[l] - row0 : TILE_ROWS);
  for (int i = tid; i < rows_here; i += SCAN_THREADS) tile[i] = make_float2(0.0f, 0.0f);
  __syncthreads();

  // ---- this slice's range of 32-point words
  const int64_t w_begin = sp.words * slice / n_slices;
  const int64_t w_end = sp.words * (slice + 1) / n_slices;
  const uint32_t* plane = sp.plane0[l] >= 0 ? planes + (int64_t)(sp.plane0[l] + (int)tile_id) * sp.words : nullptr;
  uint32_t* q = queues + wave * QUEUE_CAP;
  int qn = 0;  // wave-uniform number of queued point indices
  // One batch of 64 points is always in flight: its loads were issued when it left the queue and are
  // consumed one drain later, so memory latency overlaps the bit expansion and the previous batch's adds.
  PointData pend;
  pend.x[0] = pend.x[1] = pend.x[2] = 0.0f;
  pend.packed = 0u;  // a zero gradient makes the first (empty) batch a no-op

  for (int64_t wb = w_begin + (int64_t)wave * 64; wb < w_end; wb += (int64_t)SCAN_WAVES * 64) {
    const int64_t wi = wb + lane;
    uint32_t word = 0u;
    if (wi < w_end) {
      if (plane != nullptr) {
        word = plane[wi];
      } else {
        // single-tile level: every existing point hits
        const int64_t left = N - wi * 32;
        word = left >= 32 ? 0xffffffffu : (left > 0 ? ((1u << left) - 1u) : 0u);
      }
    }
    // each round every lane with bits left queues the point of its lowest set bit
    while (true) {
      const bool has = word != 0u;
      const unsigned long long vote = __ballot(has);
      if (vote == 0ull) break;
      if (has) {
        const int b = __ffs((int)word) - 1;
        word &= word - 1u;
        const int pos = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(vote >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)vote, 0u));
        q[qn + pos] = (uint32_t)(wi * 32 + b);
      }
      qn += __popcll(vote);
      __builtin_amdgcn_wave_barrier();
      if (qn >= 64) {
        const uint32_t n = q[qn - 64 + lane];
        qn -= 64;
        __builtin_amdgcn_wave_barrier();
        const PointData next = fetch_point<FAST>(n, coords, cdt, csn, csd, gl);
        scatter_point<GT>(tile, tile_id, pend, l, hashed, xfree, g, pi, scale);
        pend = next;
      }
    }
  }
  __builtin_amdgcn_wave_barrier();
  scatter_point<GT>(tile, tile_id, pend, l, hashed, xfree, g, pi, scale);
  if (lane < qn) {
    const PointData last = fetch_point<FAST>(q[lane], coords, cdt, csn, csd, gl);
    scatter_point<GT>(tile, tile_id, last, l, hashed, xfree, g, pi, scale);
  }
  __syncthreads();

  // ---- add the tile to the global table: consecutive lanes -> consecutive floats (16 per atomic request)
  float* dst = dtable + (g.row_offset[l] + row0) * 2;
  const float* src = reinterpret_cast<const float*>(tile);
  for (int i = tid; i < rows_here * 2; i += SCAN_THREADS) {
    const float v = src[i];
    if (v != 0.0f) unsafeAtomicAdd(dst + i, v);
  }
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------
static bool scan_applicable(const nf_hash_geom* geom, int dout_dtype) {
  if (geom->dims != 3 || geom->feat != 2 || dout_dtype == NF_F32) return false;
  for (int l = 0; l < geom->levels; ++l) {
    const int64_t r = geom->rows[l];
    if (l >= geom->first_hash_level && (r & (r - 1)) != 0) return false;  // hashed levels: power-of-two sizes
  }
  return true;
}

static void make_plan(int64_t N, const nf_hash_geom* geom, ScanPlan* sp) {
  sp->n_levels = geom->levels;
  const int64_t plan_blocks = (N + PLAN_POINTS - 1) / PLAN_POINTS;
  sp->words = plan_blocks * 32;
  int planes = 0, task = 0;
  for (int l = 0; l < geom->levels; ++l) {
    const int tiles = (int)((geom->rows[l] + TILE_ROWS - 1) / TILE_ROWS);
    sp->tiles[l] = tiles;
    const bool hashed = l >= geom->first_hash_level;
    sp->xfree[l] = hashed && (int64_t)geom->res[l] + 1 <= TILE_ROWS;
    if (tiles > 1) {
      sp->plane0[l] = planes;
      planes += tiles;
    } else {
      sp->plane0[l] = -1;
    }
    // expected share of the points that touch one tile
    double frac = 1.0;
    if (tiles > 1) frac = hashed ? (sp->xfree[l] ? 4.0 : 8.0) / tiles : 1.5 / tiles;
    if (frac > 1.0) frac = 1.0;
    const int64_t per_task = hashed && tiles > 1 ? HITS_PER_TASK_HASHED : HITS_PER_TASK_DENSE;
    int64_t slices = (int64_t)((double)N * frac / (double)per_task + 0.999);
    if (slices < 1) slices = 1;
    if (slices > 256) slices = 256;
    sp->slices[l] = (int)slices;
  }
  // segments between consecutive distinct slice counts
  int bounds[NF_MAX_LEVELS + 1];
  int nb = 0;
  for (int l = 0; l < geom->levels; ++l) {
    bool seen = false;
    for (int i = 0; i < nb; ++i) seen = seen || bounds[i] == sp->slices[l];
    if (!seen) bounds[nb++] = sp->slices[l];
  }
  for (int i = 0; i < nb; ++i)
    for (int j = i + 1; j < nb; ++j)
      if (bounds[j] < bounds[i]) {
        const int t = bounds[i];
        bounds[i] = bounds[j];
        bounds[j] = t;
      }
  int s0 = 0;
  sp->n_segs = nb;
  for (int k = 0; k < nb; ++k) {
    int width = 0;
    for (int l = 0; l < geom->levels; ++l)
      if (sp->slices[l] > s0) width += sp->tiles[l];
    sp->seg_s0[k] = s0;
    sp->seg_task0[k] = task;
    sp->seg_width[k] = width;
    task += width * (bounds[k] - s0);
    s0 = bounds[k];
  }
  sp->seg_s0[nb] = s0;
  sp->seg_task0[nb] = task;
  sp->n_tasks = task;
  sp->planes_pad = planes | 1;
}

int64_t bwd_scan_workspace_bytes(int64_t n_points, const nf_hash_geom* geom, int dout_dtype) {
  if (!scan_applicable(geom, dout_dtype) || n_points <= 0) return 0;
  ScanPlan sp;
  make_plan(n_points, geom, &sp);
  int planes = 0;
  for (int l = 0; l < geom->levels; ++l)
    if (sp.plane0[l] >= 0) planes = sp.plane0[l] + sp.tiles[l];
  if ((size_t)32 * sp.planes_pad * 4 > 150 * 1024) return 0;  // more tiles than the plan kernel's LDS holds (tables beyond 2^20 rows per level)
  // bit-planes, then the transposed gradient gT[level][point]
  return ((int64_t)planes + (int64_t)geom->levels * 32) * sp.words * 4;
}

int launch_bwd_scan(const void* coords, int cdt, int64_t csn, int64_t csd, const void* dout, int ddt, int64_t dout_stride,
                    float* dtable, int64_t N, const nf_hash_geom* geom, const DevGeom& g, const int64_t* primes, float scale,
                    void* workspace, hipStream_t s) {
  ScanPlan sp;
  make_plan(N, geom, &sp);
  int planes = 0;
  for (int l = 0; l < geom->levels; ++l)
    if (sp.plane0[l] >= 0) planes = sp.plane0[l] + sp.tiles[l];
  uint32_t* planes_w = (uint32_t*)workspace;
  uint32_t* gT = planes_w + (int64_t)planes * sp.words;
  {
    const size_t lds = (size_t)32 * sp.planes_pad * 4;
    NF_REQUIRE(lds <= 150 * 1024, NF_EUNSUPPORTED, "%d tiles need %zu B of LDS in the plan kernel", planes, lds);
    if (lds > 64 * 1024) {
      hipError_t e = hipFuncSetAttribute((const void*)hash_bwd_plan_k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    }
    hipLaunchKernelGGL(hash_bwd_plan_k, dim3((unsigned)(sp.words / 32)), dim3(PLAN_POINTS), lds, s, coords, cdt, csn, csd,
                       (const uint16_t*)dout, dout_stride, planes_w, gT, N, g, sp, primes, scale);
    if (int rc = check_launch("hash_bwd_plan")) return rc;
  }
  const size_t lds = (size_t)TILE_ROWS * sizeof(float2) + (size_t)SCAN_WAVES * QUEUE_CAP * 4;
  const int tasks = sp.n_tasks;
  const bool fast = cdt == NF_F32 && csn == 3 && csd == 1 && scale == 1.0f && N * 3 < ((int64_t)1 << 31);
  const void* kern = nullptr;
  if (ddt == NF_F16)
    kern = fast ? (const void*)hash_bwd_scan_k<F16, true> : (const void*)hash_bwd_scan_k<F16, false>;
  else
    kern = fast ? (const void*)hash_bwd_scan_k<BF16, true> : (const void*)hash_bwd_scan_k<BF16, false>;
  hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return fail((int)e, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  const uint32_t* planes_c = planes_w;
  const uint32_t* gT_c = gT;
  void* args[] = {(void*)&coords, (void*)&cdt, (void*)&csn, (void*)&csd, (void*)&gT_c, (void*)&dtable,
                  (void*)&planes_c, (void*)&N, (void*)&g, (void*)&sp, (void*)&primes, (void*)&scale};
  e = hipLaunchKernel(kern, dim3((unsigned)tasks), dim3(SCAN_THREADS), args, lds, s);
  if (e != hipSuccess) return fail((int)e, "hipLaunchKernel(hash_bwd_scan): %s", hipGetErrorString(e));
  return check_launch("hash_bwd_scan");
}

}  // namespace nf
