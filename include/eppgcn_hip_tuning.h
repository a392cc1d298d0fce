/*
 * Tuning and test knobs of libeppgcn_hip.so.  Not part of the drop-in surface: nothing in the
 * reference corresponds to them, and a product build never needs to call any of them.
 *
 * Every setter here writes a PROCESS-WIDE value (an atomic word, so a setter that races with a call is
 * not a data race - but the call may see either value): it changes the launches of every thread of the
 * process from the next call on, so set them before the calls they are meant for, from one place.  They exist for benchmark sweeps and for tests that have to reach code paths a
 * small input would not (64-bit indexing, a stalled look-back, the group kernel over a plan).
 */
#ifndef EPPGCN_HIP_TUNING_H_
#define EPPGCN_HIP_TUNING_H_

#include "eppgcn_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* 0 keeps every planned call on the group kernel (for comparisons); 1 (default) allows the stream form;
 * 2 allows it and forces its 64-bit addressing variant at any table size (for tests: it otherwise runs
 * for tables of 4 GB and more).  Set it before the plans are built: the order of a plan follows the
 * kernel that will run over it. */
void eppgcn_set_stream_mode(int on);
/* Forces the number of lanes per neighbour group in the aggregation kernels
 * (power of two in 4..64; 0 = choose from the feature width).  For tuning runs. */
void eppgcn_set_team_size(int lanes);
/* Forces the number of consecutive group rounds one wave processes (0 = choose from
 * the group size so that a wave gathers about 512 rows).  For tuning runs. */
void eppgcn_set_rounds(int rounds);
/* The output-clear and pre-scaling kernels index with 32 bits while the matrices have fewer than 2^32
 * elements; 1 forces their 64-bit instantiations at any size.  For tests. */
void eppgcn_set_wide_index(int on);
/* For tests of the stall path of the look-back scans: spin_limit > 0 replaces the number of polls after
 * which a waiting tile gives up (default 2^22); mute_first_tile != 0 makes tile 0 of every scan keep its
 * result to itself, so that every later tile runs into the limit, raises the stall flag and carries on
 * with what it has - the kernels still finish, the results are invalid, and the calls that read the
 * status return EPPGCN_ERR_SCAN_STALLED.  (0, 0) restores normal operation. */
void eppgcn_set_scan_test_mode(unsigned spin_limit, int mute_first_tile);
/* Forces the column block size of eppgcn_build_plan to 2^shift vertices (0 = choose from the
 * feature width).  For tuning runs. */
void eppgcn_set_plan_shift(int shift);
/* Plan policy (tuning runs).  Rows of at most 32 * groups slots (and at most 64 groups) stay together in
 * a plan instead of being cut at column-block borders (0 = block every group).  Negative (the default) =
 * chosen per build: 2 when the launch shape (num_nodes, dim) is one the stream form runs, 8 when the
 * group kernel will run over the plan. */
void eppgcn_set_plan_keep_rows(int groups);
/* Within a column block, order single-group rows by length class (1-8, 9-16, 17-24, 25+ slots) so
 * that the groups of one round take the same number of gather steps.  1 on, 0 off, negative (the
 * default) = per build: off for the stream form (its gather instructions are full whatever the
 * lengths), on for the group kernel. */
void eppgcn_set_plan_length_classes(int on);

#ifdef __cplusplus
}
#endif
#endif /* EPPGCN_HIP_TUNING_H_ */
