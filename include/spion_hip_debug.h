/*
 * spion_hip_debug.h -- testing and profiling aids of libspion_hip.so.  Not product surface: nothing in a
 * deployment needs them; the test-suite and the benchmark use them to compare kernel families and to time the
 * two backward kernels separately.  No counterpart in the reference.
 */
#ifndef SPION_HIP_DEBUG_H
#define SPION_HIP_DEBUG_H

#ifdef __cplusplus
extern "C" {
#endif

/* Force the element path even for tile-structured patterns (testing / comparison).  Drops every analysed
 * pattern of the handle. */
void spion_force_element_path(void* handle, int on);

/* Run only part of a sparse handle's backward.  bit 0 = row pass (row sums and dQ), bit 1 = column pass (dK, dV;
 * needs the row sums of an earlier row pass).  Default 3 = both. */
void spion_set_backward_passes(void* handle, int mask);

/* Counters of a sparse handle: which = 0 -> pattern analyses that copied the index back from the device (and
 * waited for the stream), which = 1 -> analyses made from host arrays (spion_register_pattern), which = 2 ->
 * workspace buffers that a larger pattern has outgrown and that stay allocated until the handle is destroyed (a HIP
 * graph recorded before the growth still points at them).  -1 otherwise. */
int spion_debug_counter(void* handle, int which);

/* The schedule the bf16 kernels would walk for a tile list (host only: needs no device).  tile_ptr[nstrips + 1]: first
 * tile of every 32-row (or 32-column) strip; pairs != 0: strips 2p and 2p+1 hold the same tiles and are walked
 * together; lanes: persistent wavefronts asked for.  Returns the number of lanes the schedule uses (-1 on bad
 * arguments) and fills, where the arrays are large enough (cap_* in ints):
 *   items     {strip, first tile, tiles, kind} per item -- kind >= 0: chunk of a long strip, its workspace slot;
 *             -1: whole strip; -2: the pair (strip, strip + 1);
 *   lane_ptr  [lanes + 1], lane_ent {head, item} per entry: lane s walks entries lane_ptr[s] .. lane_ptr[s+1]-1;
 *   longs     {strip, first slot, chunks, tiles} per long strip;
 *   counts    {ints in items, ints in lane_ent, ints in longs, workspace slots}. */
int spion_debug_bf16_plan(const int* tile_ptr, int nstrips, int pairs, int num_batches, int lanes, int* items,
                          int cap_items, int* lane_ptr, int cap_ptr, int* lane_ent, int cap_ent, int* longs,
                          int cap_longs, int* counts);

/* Environment switches read once per process, for A/B measurements only (results are the same to rounding either way):
 *   SPION_NO_FWD_SPLIT   the fp32 tile forward runs all strips in one launch, eight logit tiles per wavefront
 *                        (default: strips of at most 16 tiles in a launch of their own, three work-groups to a CU);
 *   SPION_NO_LONG_SPLIT  patterns with a few strips far longer than the rest (global rows / columns) run every pass of
 *                        the fp32 tile path as one launch with four wavefronts to every strip (default: the long strips
 *                        in a launch of their own on the caller's stream, the others beside it on the handle's side
 *                        stream; the summation order inside the short strips differs between the two);
 *   SPION_BF16_NO_PAIRS  the bf16 forward and row pass take one strip per wavefront on every pattern (default: two
 *                        strips per wavefront on masks of 64 x 64 blocks and larger, contiguous heads);
 *   SPION_BF16_ROW_PAIRS=0  the same for the row pass alone.
 *   SPION_HYB_GATHER     hybrid patterns: the remainder's column pass gathers its Q and dO rows from L2, one wavefront
 *                        per column (default, when seq_len is a multiple of 1024 and num_batches * seq_len / 256 >= 256:
 *                        work-groups of 1024, 512 or 256 columns with the rows of a range of the sequence in LDS; the
 *                        element kernels' column pass at emb_dim 32 likewise), and so do the forward's two remainder
 *                        kernels (default: operands in LDS when num_batches * seq_len / 512, resp. / 1024, >= 256);
 * Read whenever a bf16 handle indexes a pattern (tests):
 *   SPION_BF16_LANES     number of persistent wavefronts the bf16 kernels are launched with (default: eight per
 *                        compute unit); a handful makes each one walk many strips of several heads in a row.
 * Read once, at the first sparse call:
 *   SPION_ROCTX=1        roctx ranges around the phases of every sparse call ("spion forward (tile kernels)",
 *                        "spion backward: row pass (dQ)", "spion backward: column pass (dK, dV)", ...: the host-side
 *                        intervals in which the phase's kernels are enqueued), as the reference brackets its cuSPARSE
 *                        steps with nvtx ranges (models/block_attn.cu:163-223); `rocprofv3 --marker-trace` shows
 *                        them.  The tools library is loaded with dlopen only when the switch is set.
 * SPION_QUIET and SPION_ABORT_ON_ERROR (error reporting) are described in spion_hip.h. */

#ifdef __cplusplus
}
#endif
#endif /* SPION_HIP_DEBUG_H */
