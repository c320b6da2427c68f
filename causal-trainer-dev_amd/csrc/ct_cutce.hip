// placeholder until the cut cross-entropy kernels land
#include "ct_error.h"
extern "C" size_t ct_cutce_fwd_workspace_bytes(const ct_cutce_shape*) { return 0; }
extern "C" size_t ct_cutce_bwd_workspace_min_bytes(const ct_cutce_shape*) { return 0; }
extern "C" size_t ct_cutce_bwd_workspace_bytes(const ct_cutce_shape*) { return 0; }
extern "C" int32_t ct_cutce_fwd(void*, const ct_cutce_fwd_args*) { return ct::fail(CT_UNSUPPORTED, "not built yet"); }
extern "C" int32_t ct_cutce_bwd(void*, const ct_cutce_bwd_args*) { return ct::fail(CT_UNSUPPORTED, "not built yet"); }
