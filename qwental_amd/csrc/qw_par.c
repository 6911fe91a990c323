// The cut of a step into launches from measured times (include/qw_par.h). Plain host arithmetic, no GPU call.
#include "qw_par.h"
#include <stdlib.h>

#define NBUCKET (QW_PAR_PACK_MAX / 16)

struct qw_par {
    double cost[QW_PAR_VBMAX + 1];
    int seen[QW_PAR_VBMAX + 1];
    double pcost[NBUCKET + 1]; // bucket k: rows 16 (k - 1) + 1 .. 16 k
    int pseen[NBUCKET + 1];
};

qw_par *qw_par_new(void) { return calloc(1, sizeof(qw_par)); }
void qw_par_free(qw_par *p) { free(p); }

// src/engine.c:9037: the first sample of a size is dropped, the second starts the average, later ones move it by a tenth
static void observe(double *cost, int *seen, double ms) {
    if ((*seen)++) *cost = *cost > 0 ? 0.9 * *cost + 0.1 * ms : ms;
}
void qw_par_observe(qw_par *p, int b, double ms) {
    if (b >= 1 && b <= QW_PAR_VBMAX && ms > 0) observe(&p->cost[b], &p->seen[b], ms);
}
double qw_par_group_cost(const qw_par *p, int b) { return b >= 1 && b <= QW_PAR_VBMAX ? p->cost[b] : 0; }

// Sizes never measured, filled in on the line through the smallest and the largest measured size (one size: flat).
// Two measured sizes close together can give the line any slope (a launch's time varies by a few per cent): a falling
// line is taken as flat at the cheapest measured size, and no size is estimated below half of that, so that an estimate is never
// zero or negative (a step cut into many groups that "cost nothing").
static bool fill_line(const double *c, int n, double *out) {
    int lo = 0, hi = 0;
    double least = 0;
    for (int b = 1; b <= n; b++)
        if (c[b] > 0) {
            if (!lo) lo = b;
            hi = b;
            if (least == 0 || c[b] < least) least = c[b];
        }
    if (!lo) return false;
    double a = hi > lo ? least : c[lo], k = 0;
    if (hi > lo && c[hi] > c[lo]) {
        k = (c[hi] - c[lo]) / (hi - lo);
        a = c[lo] - k * lo;
    }
    for (int b = 1; b <= n; b++) {
        out[b] = c[b] > 0 ? c[b] : a + k * b;
        if (out[b] < 0.5 * least) out[b] = 0.5 * least;
    }
    return true;
}

// One dynamic programme serves both questions (src/engine.c:8764-8797). cheapest[n]: least total of group costs c[]
// that covers n rows; last[n]: the size of the group that completes it. Among equal totals the larger group wins.
static void cover(const double *c, int B, double *cheapest, int *last) {
    cheapest[0] = 0;
    for (int n = 1; n <= B; n++) {
        cheapest[n] = 1e30;
        last[n] = 1;
        for (int b = 1; b <= QW_PAR_VBMAX && b <= n; b++) {
            const double total = cheapest[n - b] + c[b];
            if (total <= cheapest[n]) cheapest[n] = total, last[n] = b;
        }
    }
}

double qw_par_cost(const qw_par *p, int B) { // the estimate: sizes never measured lie on the line through the measured ones
    if (B < 1) return 0;
    double c[QW_PAR_VBMAX + 1], cheapest[QW_PAR_MAX + 1];
    int last[QW_PAR_MAX + 1];
    if (!fill_line(p->cost, QW_PAR_VBMAX, c)) return 0;
    if (B > QW_PAR_MAX) B = QW_PAR_MAX;
    cover(c, B, cheapest, last);
    return cheapest[B];
}

int qw_par_split(const qw_par *p, int B, int *g) { // the cut: a size never measured costs 0, so that it gets tried
    if (B < 1 || B > QW_PAR_MAX) return 0;
    double cheapest[QW_PAR_MAX + 1];
    int last[QW_PAR_MAX + 1], ng = 0;
    cover(p->cost, B, cheapest, last);
    for (int n = B; n > 0; n -= last[n]) g[ng++] = last[n];
    return ng;
}

static int bucket(int rows) { return (rows + 15) / 16; }
void qw_par_observe_packed(qw_par *p, int rows, double ms) {
    if (rows >= 1 && rows <= QW_PAR_PACK_MAX && ms > 0) observe(&p->pcost[bucket(rows)], &p->pseen[bucket(rows)], ms);
}
double qw_par_packed_cost(const qw_par *p, int rows) {
    if (rows < 1) return 0;
    double c[NBUCKET + 1];
    if (!fill_line(p->pcost, NBUCKET, c)) return 0;
    const int k = bucket(rows > QW_PAR_PACK_MAX ? QW_PAR_PACK_MAX : rows);
    return c[k];
}

bool qw_par_choose(const qw_par *p, int rows, int *groups, int *ngroups) {
    *ngroups = rows <= QW_PAR_MAX ? qw_par_split(p, rows, groups) : 0;
    if (rows < 1) return false;
    // the grouped form beyond QW_PAR_MAX rows: full steps of QW_PAR_MAX rows plus the rest
    double grouped = 0;
    for (int left = rows; left > 0; left -= QW_PAR_MAX) {
        const double c = qw_par_cost(p, left > QW_PAR_MAX ? QW_PAR_MAX : left);
        if (c <= 0) return false;
        grouped += c;
    }
    const double packed = qw_par_packed_cost(p, rows);
    return packed > 0 && packed < grouped;
}

// tools/serve.c:1715-1729 of the reference. Two ways to serve n conversations that are decoding: one at a time in time
// slices (each runs at its own speed, speculative decoding included, and pays for the switches), or all together as one
// step of n rows. Rates in tokens per second; 0 = not measured.
bool qw_par_want_slice(const qw_par *p, int n, bool slicing_now, double sliced_rate, const double *solo_rate, double solo_default, double batched_rate) {
    if (n <= 1) return true;
    if (n > QW_PAR_SLICE_MAX) return false;
    double rs = sliced_rate;
    if (rs <= 0) { // never measured with the switches in: the mean of what each conversation reaches inside its own slice
        rs = 0;
        for (int i = 0; i < n; i++) rs += solo_rate && solo_rate[i] > 0 ? solo_rate[i] : solo_default;
        rs /= n;
    }
    double rb = batched_rate;
    if (rb <= 0) { // never measured: n rows per estimated step
        const double ms = qw_par_cost(p, n);
        rb = ms > 0 ? n * 1e3 / ms : 0;
    }
    if (rs <= 0 || rb <= 0) return false; // no figures: together (with two or more that is usually the faster way)
    return rs > rb * (slicing_now ? 0.95 : 1.05); // five per cent either way before the mode changes
}
