/* The header is plain C: this file is compiled with a C compiler (-std=c11 -pedantic -Werror) and
 * linked against libfv_sdpa_hip.so; it calls host-only entry points (no GPU needed) and prints what
 * the test compares against the reference's known answers. */
#include <stdio.h>
#include <string.h>

#include "fv_sdpa_hip.h"

int main(void) {
    size_t dims[5], mv[4], bc[3], ranges[4];
    int steps[4], n_steps;
    const size_t shape[4] = {1, 12, 320, 128};
    fv_tensor t;
    fv_plan p;
    memset(&t, 0, sizeof t);
    memset(&p, 0, sizeof p);
    p.kind = FV_PLAN_KV_WINDOW;
    t.plane_rows = 0;
    if (strcmp(fv_sdpa_arch(), "gfx950") != 0) return 1;
    if (fv_vsa_tile_plan(21, 30, 52, dims, NULL, NULL, NULL) != FV_OK) return 2;
    if (fv_kv_plan(60, 10, 60, 10, 1, 60, 60, 60, 30, mv) != FV_OK) return 3;
    if (fv_kv_plan(210, 0, 210, 10, 0, 210, 210, 210, 10, mv + 0) == FV_OK) return 4;   /* a 22nd frame is refused */
    if (fv_kv_plan(60, 10, 60, 10, 1, 60, 60, 60, 30, mv) != FV_OK) return 5;
    if (!fv_block_causal_for(3, 6, 390, bc)) return 6;
    fv_sp_shard_ranges(11, 2, ranges);
    n_steps = fv_rt_dense_route(shape, shape, shape, 0, 0, steps, NULL);
    printf("supported=%d%d tiles=%zu topk=%zu kvmove=%zu,%zu,%zu,%zu block_causal=%zu,%zu,%zu shards=%zu,%zu,%zu,%zu "
           "backend=%d route=%d:%d,%d err=\"%s\"\n",
           fv_sdpa_supported(1, 12, 32760, 32760, 128), fv_sdpa_supported(1, 12, 32760, 32760, 96),
           dims[0] * dims[1] * dims[2], fv_vsa_topk_for(0.8, dims[0] * dims[1] * dims[2]), mv[0], mv[1], mv[2], mv[3],
           bc[0], bc[1], bc[2], ranges[0], ranges[1], ranges[2], ranges[3], fv_rt_parse_backend("cublas"),
           n_steps, steps[0], steps[1], fv_sdpa_last_error());
    return 0;
}
