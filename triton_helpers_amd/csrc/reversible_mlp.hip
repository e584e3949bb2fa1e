#include "nf_common.h"
extern "C" int nf_revmlp_fwd(const void*, int64_t, void*, int64_t, const void*, const void*, const void*, const void*, int64_t, int, int, int, int, void*) { return nf::fail(NF_EUNSUPPORTED, "nf_revmlp_fwd not built yet"); }
extern "C" int nf_revmlp_bwd(const void*, int64_t, const void*, int64_t, void*, int64_t, void*, int64_t, const void*, const void*, const void*, const void*, float*, float*, float*, float*, int64_t, int, int, int, int, void*) { return nf::fail(NF_EUNSUPPORTED, "nf_revmlp_bwd not built yet"); }
