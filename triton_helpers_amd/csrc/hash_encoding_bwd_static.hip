// nf_hash_encode_bwd_static: the hash-encoding backward for callers that cannot allocate device memory (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It is nf_hash_encode_bwd with the
// scratch of its sort-and-accumulate kernels taken from a device array that lives in this library instead of a
// caller's workspace: nothing is allocated or freed, on the device or on the host.
//
// The array is NF_HASH_BWD_STATIC_BYTES large on every GPU the library is loaded on and stays until the process ends.
// Its device address differs per GPU and is asked for once per device (hipGetSymbolAddress with that device
// current); host code never uses the array's name for anything else.  All calls on one GPU share the array: calls that
// overlap in time on one GPU (two streams, two threads) race on it.  The kernels clear what they need cleared
// themselves (with a fill kernel, not a memset node), so the previous call's contents do not matter.
#include <atomic>

#include "hash_common.h"

namespace nf {

static __device__ __attribute__((used)) __align__(256) unsigned char scratch[NF_HASH_BWD_STATIC_BYTES];

// scratch's address on the current device (cached per device ordinal; racing first calls ask twice and agree)
static int static_scratch(void** out) {
  static std::atomic<void*> cached[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail((int)e, "hipGetDevice: %s", hipGetErrorString(e));
  NF_REQUIRE(dev >= 0 && dev < 64, NF_EUNSUPPORTED, "device ordinal %d beyond the 64 this entry point keeps addresses for", dev);
  void* p = cached[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) return fail(e != hipSuccess ? (int)e : NF_EINVAL, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    cached[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return 0;
}

}  // namespace nf

using namespace nf;

extern "C" int64_t nf_hash_encode_bwd_static_bytes(void) { return (int64_t)NF_HASH_BWD_STATIC_BYTES; }

extern "C" int nf_hash_encode_bwd_static(const void* coords, int coords_dtype, int64_t csn, int64_t csd, const void* dout,
                                         int dout_dtype, int64_t dout_stride_n, float* dtable, int64_t n_points,
                                         const nf_hash_geom* geom, const int64_t* primes, float scale, int flags, void* stream) {
  NF_REQUIRE(geom != nullptr, NF_EINVAL, "geom is NULL");
  NF_REQUIRE(n_points >= 0, NF_EINVAL, "n_points negative");
  // Which variant's scratch fits: the sorted records (fastest, ~1.5 KB per point), else the bit-planes (~110 B per
  // point, 16-bit gradients of 3-D points only).  A call that would need neither (small batches and shapes that
  // scatter with atomics) needs no scratch at all.
  const int64_t limit = (int64_t)NF_HASH_BWD_STATIC_BYTES;
  const int64_t need_bin = nf_hash_encode_bwd_workspace_bytes(n_points, geom, dout_dtype, flags & ~NF_HASH_FORCE_PLANES);
  const int64_t need_planes = nf_hash_encode_bwd_workspace_bytes(n_points, geom, dout_dtype, flags | NF_HASH_FORCE_PLANES);
  int use_flags = flags;
  if (need_bin > limit || (flags & NF_HASH_FORCE_PLANES)) {
    NF_REQUIRE(need_planes > 0 && need_planes <= limit, NF_EINVAL,
               "n_points=%lld needs %lld bytes of scratch (%lld with the bit-plane variant, 0 = not applicable to this call); "
               "the static scratch holds %lld: split the batch or call nf_hash_encode_bwd with a workspace",
               (long long)n_points, (long long)need_bin, (long long)need_planes, (long long)limit);
    use_flags |= NF_HASH_FORCE_PLANES;
  }
  void* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  return nf_hash_encode_bwd(coords, coords_dtype, csn, csd, dout, dout_dtype, dout_stride_n, dtable, n_points, geom, primes, scale, ws,
                            limit, use_flags, stream);
}
