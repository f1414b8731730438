// Ragged causal prefill attention for gfx950.
#include <new>
#include "bz_common.hpp"

namespace bz {
struct PrefillPlan {
    bool planned = false;
    uint32_t batch_size = 0, num_qo_heads = 0, num_kv_heads = 0, head_dim = 0;
};
} // namespace bz
using namespace bz;

extern "C" bz_prefill_plan_t* bz_prefill_plan_create(void) {
    return reinterpret_cast<bz_prefill_plan_t*>(new (std::nothrow) PrefillPlan());
}
extern "C" void bz_prefill_plan_destroy(bz_prefill_plan_t* p) { delete reinterpret_cast<PrefillPlan*>(p); }
extern "C" int bz_prefill_plan(bz_prefill_plan_t*, void*, size_t, void*, size_t, const int32_t*, const int32_t*,
                               uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, void*) {
    return BZ_ERR_UNSUPPORTED;
}
extern "C" int bz_batch_prefill_ragged(bz_prefill_plan_t*, void*, const int32_t*, void*, void*, const int32_t*, void*,
                                       int, uint32_t, uint32_t, uint32_t, uint32_t, int, int, float, float, void*) {
    return BZ_ERR_UNSUPPORTED;
}
