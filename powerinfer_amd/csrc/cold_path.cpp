// Host (CPU) share of hybrid layers.  See cold_path.hpp.
#include "cold_path.hpp"
#include "engine_internal.hpp"
#include "runtime.hpp"

namespace pi {

struct ColdPath { int unused; };

ColdPath * cold_create(pi_model *) {
    set_error("hybrid (hot/cold split) layers are not available in this build");
    return nullptr;
}
void cold_destroy(ColdPath * c) { delete c; }
int cold_layer_merge(ColdPath *, int, pi_model *, hipStream_t) { return fail(PI_E_UNSUPPORTED, "hybrid layers are not available in this build"); }

}  // namespace pi
