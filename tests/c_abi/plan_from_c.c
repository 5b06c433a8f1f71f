/* A C (not C++) caller of the library: includes the public header as C, links against
 * libigs_hip.so and asks for a launch plan.  Prints the fields the Python test compares. */
#include <stdio.h>

#include "igs_hip.h"

int main(void) {
    igs_gs2d_plan_t p;
    int rc = igs_gs2d_plan(16, 8192, 256, 256, 3, IGS_GRID_SEPARABLE, &p);
    if (rc != IGS_OK) {
        fprintf(stderr, "plan failed: %s\n", igs_status_string(rc));
        return 1;
    }
    printf("%d %d %d %d %llu %llu %llu %llu\n", igs_abi_version(), (int)p.n_padded, (int)p.rec_stride,
           (int)p.bwd_tiles, (unsigned long long)p.packed_bytes, (unsigned long long)p.fwd_ws_bytes,
           (unsigned long long)p.pix_bytes, (unsigned long long)p.partial_bytes);
    rc = igs_gs2d_plan(0, 1, 1, 1, 3, IGS_GRID_GENERAL, &p);
    printf("%d %s\n", rc, igs_status_string(rc));
    return 0;
}
