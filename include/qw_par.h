/* How a step of B rows is cut into launches: the caller contract of the decode step.
 *
 * The reference cuts B concurrent conversations into groups of at most VBMAX = 8 rows, each group reading the weights
 * once, and picks the cut from measured step times (src/engine.c:8762-8797, 9037):
 *     par_cost[b], par_seen[b]   wall ms of a group of b rows, exponential average 0.9 / 0.1; the first sample of a
 *                                size is dropped (it contains the kernel build)                qw_par_observe()
 *     qw_engine_par_cost()       estimate for B rows under the best cut; sizes never measured
 *                                are filled in on the line through the smallest and largest
 *                                measured size                                                  qw_par_cost()
 *     par_split()                dynamic programme over group sizes; equal cost -> the larger
 *                                group; a size never measured counts as free (it gets tried)    qw_par_split()
 * Here a group holds up to 16 rows (the kernels' native step), and a step of many rows has a second form, the packing
 * path (every routed expert read once for all rows): qw_par_observe_packed() / qw_par_choose() weigh it against the
 * best cut with the same kind of measured table, in buckets of 16 rows.
 */
#pragma once
#include <stdbool.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { QW_PAR_VBMAX = 16, QW_PAR_MAX = 64 }; /* rows of one group; rows of one step (src/engine.h:79) */
enum { QW_PAR_PACK_MAX = 256 };             /* rows the packed form is tracked for */
enum { QW_PAR_SLICE_MAX = 3 };              /* conversations up to which time slices are weighed against a joint step (tools/serve.c:1252) */

typedef struct qw_par qw_par;

qw_par *qw_par_new(void);
void qw_par_free(qw_par *p);
/* One measured group of b rows (1 .. QW_PAR_VBMAX) took ms. */
void qw_par_observe(qw_par *p, int b, double ms);
/* The table entry of size b: the running average, 0 when not measured yet. */
double qw_par_group_cost(const qw_par *p, int b);
/* Estimated ms of a step of B rows (B above QW_PAR_MAX counts as QW_PAR_MAX); 0 when nothing was measured or B < 1. */
double qw_par_cost(const qw_par *p, int B);
/* Group sizes for B rows (1 .. QW_PAR_MAX) into groups[], from the back as the reference emits them; returns their
 * number, 0 when B is out of range. */
int qw_par_split(const qw_par *p, int B, int *groups);
/* One measured pass of the packing path over rows rows (1 .. QW_PAR_PACK_MAX). */
void qw_par_observe_packed(qw_par *p, int rows, double ms);
/* Estimated ms of the packing path for rows rows; 0 when it was never measured. */
double qw_par_packed_cost(const qw_par *p, int rows);
/* true: run the step through the packing path; false: as qw_par_split() says (groups / ngroups receive the cut when
 * rows <= QW_PAR_MAX, else ngroups = 0 and the caller cuts into full groups). The packing path is chosen only when
 * both forms have estimates and its estimate is lower. */
bool qw_par_choose(const qw_par *p, int rows, int *groups, int *ngroups);
/* The server's rule between time slices and a joint step for n decoding conversations (tools/serve.c:1715-1729 of the
 * reference, want_slice): true = one conversation at a time. n <= 1: true; n > QW_PAR_SLICE_MAX: false. sliced_rate: the
 * measured total rate of n conversations taking turns, switches included (0: not measured; then the mean of solo_rate[i],
 * each conversation's rate inside its own slice, solo_default standing in for a 0 or for solo_rate == NULL).
 * batched_rate: the measured total rate of a joint step of n rows (0: not measured; then n rows per qw_par_cost(p, n)).
 * Without a figure on either side: false. Otherwise the mode changes only when the other one is five per cent faster:
 * slicing_now keeps slices while sliced > 0.95 batched, a joint step goes over to slices only when sliced > 1.05 batched. */
bool qw_par_want_slice(const qw_par *p, int n, bool slicing_now, double sliced_rate, const double *solo_rate, double solo_default, double batched_rate);

#ifdef __cplusplus
}
#endif
