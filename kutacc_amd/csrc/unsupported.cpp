// Link-compatibility stubs.  The Kunpeng library exports more operators than this backend implements
// (reference include/kutacc.h:55-74, 266-280, 367-388).  A program linked against that library must
// still resolve those names, so each is exported here with C linkage; calling one reports "not implemented" through the usual
// KUTACC_CHECK channel (stderr line + sticky error flag) and touches none of its arguments.
// With C linkage the parameter lists do not take part in symbol resolution, hence the opaque ones.
#include "check.h"
#include "kutacc.h"

#define KUTACC_UNSUPPORTED(name)                                                          \
    extern "C" kutacc_export void name(...)                                               \
    {                                                                                     \
        KUTACC_CHECK(false, #name ": not implemented on the MI355X gated-attention backend"); \
    }

KUTACC_UNSUPPORTED(kutacc_comm_init)
KUTACC_UNSUPPORTED(kutacc_comm_fini)
KUTACC_UNSUPPORTED(kutacc_af2_transpose)
KUTACC_UNSUPPORTED(kutacc_af2_all_gather)
KUTACC_UNSUPPORTED(kutacc_af2_outer_product_mean_calc_left_and_right_mul)
KUTACC_UNSUPPORTED(kutacc_af2_outer_product_mean_chunk)
KUTACC_UNSUPPORTED(kutacc_af2_invariant_point)
KUTACC_UNSUPPORTED(kutacc_af2_rigid_rot_vec_mul)
KUTACC_UNSUPPORTED(kutacc_af2_rigid_rot_matmul)
