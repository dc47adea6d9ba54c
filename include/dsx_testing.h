/* dsx_testing.h — switches of libdsx_hip.so that exist for its tests: they make small inputs reach the code paths that
 * otherwise only large ones take.  Not part of the drop-in boundary (include/dsx.h) and without counterpart in the reference.
 * Results never depend on them.  The values live in the library's context: dsx_shutdown (the last one) and dsx_testing_reset
 * put every switch back to its default; like every call of the library they belong to the one thread that drives it. */
#ifndef DSX_TESTING_H
#define DSX_TESTING_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* Rows of a workgroup's tile in dsx_fc_forward_split: 128 or 256; 0 (default) chooses by shape. */
int dsx_testing_set_split_tile_rows(uint32_t rows);
/* dsx_fc_topk: width of the first column block (0: default 2,048; at most 131,072) and survivor words per row and column range
 * (64 .. 4,096; 0: default 4,096). */
int dsx_testing_set_fc_topk_first_columns(uint32_t columns);
int dsx_testing_set_fc_topk_candidate_capacity(uint32_t words);
/* dsx_knn_search*: width of the first column block (rounded down to a multiple of 1024, at least 1024; 0 restores the default
 * of about 1 GiB of scores).  Workspace sizes depend on it: set it before asking for them. */
int dsx_testing_set_knn_block_columns(uint32_t columns);
/* dsx_knn_search_f16, column ranges after the first block.  1 (default): swept by workgroups that keep their queries when the
 * range is long enough; 0: always one workgroup per tile; 2 and 3: the LDS sweep and the register sweep for every range that
 * has at least one tile per chunk. */
int dsx_testing_set_knn_f16_sweep(int mode);
/* Occupancy probe: launches `workgroups` workgroups of 256 lanes on the selected lane that do nothing but hold their place for
 * about `cycles` shader clocks (bounded; every wavefront exits), with 128, 64 or (any other value) next to no vector
 * registers per lane.  bench.py --interference uses it to separate what a kernel beside a dense layer costs that layer by
 * merely being resident from what its instructions and memory traffic cost. */
int dsx_testing_occupy(uint32_t workgroups, uint32_t cycles, uint32_t vgprs);
/* Every switch back to its default. */
int dsx_testing_reset(void);

#ifdef __cplusplus
}
#endif
#endif /* DSX_TESTING_H */
