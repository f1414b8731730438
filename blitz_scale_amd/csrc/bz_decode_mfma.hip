// MFMA decode path for gfx950 (placeholder until the tiled kernel lands: everything is routed to
// the general kernel).
#include "bz_common.hpp"
#include "bz_decode_plan.hpp"

namespace bz {
struct DecodeArgs;
int decode_fast_path(const DecodePlan*, const DecodeArgs&, int, int, int, int, int, const bz_paged_kv_t*,
                     hipStream_t) {
    return BZ_ERR_UNSUPPORTED;
}
} // namespace bz
