// How a product's result Y [M, N] is cut into tiles for the kernels that hold one workgroup of eight wavefronts a
// compute unit (qgemm_f16_panel.hip, qgemm_q4_0_blocks.hip): a compute unit takes the next tile when it is free, so a
// product takes as long as the unit with the most tiles, and where tiles of 256 x 256 would leave the last round partly
// empty the right-hand columns are cut into tiles of 256 x 192 instead, handed out after the wide ones; products with too
// few wide tiles for the device take tiles of 128 x 256. The cut is chosen by the time the last tile ends.
#pragma once
#include <cstdint>

namespace mimir {

constexpr int kUnits = 256;  // compute units; one workgroup each at a time (LDS)

// Columns [0, 256 wide_cols) in tiles of 256 x 256, then narrow_cols tiles of 256 x 192 a row of tiles; or, with `low`,
// every tile 128 x 256. Workgroups take the wide tiles first (the dispatcher hands them out in the order of their index).
struct PanelPlan {
    int tiles_m;      // tiles along M (256 rows, or 128 with low)
    int wide_cols, narrow_cols;
    int low;
};

// When the last of n_first jobs of cost c_first, then n_then jobs of cost c_then, ends on kUnits units that each
// take the next job as soon as they are free.
inline double makespan(int n_first, double c_first, int n_then, double c_then) {
    struct Level { double at; int units; };
    Level lv[64];
    int n = 0;
    const int q = n_first / kUnits, r = n_first % kUnits;
    if (kUnits - r > 0) lv[n++] = {q * c_first, kUnits - r};
    if (r > 0) lv[n++] = {(q + 1) * c_first, r};
    while (n_then > 0) {
        const int k = lv[0].units < n_then ? lv[0].units : n_then;  // lv is kept in ascending order
        n_then -= k;
        const double to = lv[0].at + c_then;
        lv[0].units -= k;
        if (lv[0].units == 0) {
            for (int i = 1; i < n; i++) lv[i - 1] = lv[i];
            n--;
        }
        int at = 0;
        while (at < n && lv[at].at < to) at++;
        if (at < n && lv[at].at == to) {
            lv[at].units += k;
        } else if (n < 64) {
            for (int i = n; i > at; i--) lv[i] = lv[i - 1];
            lv[at] = {to, k};
            n++;
        } else {
            lv[n - 1].units += k;  // more levels than this holds: counted at the latest
        }
    }
    return n > 0 ? lv[n - 1].at : 0.0;
}

// The cut with the earliest end, and that end, in wide tiles' time; narrow_cost and low_cost: what a tile of 256 x 192 and
// one of 128 x 256 take of it.
inline double plan_panel(int64_t M, int64_t N, double narrow_cost, double low_cost, PanelPlan* out) {
    const int tm = (int)((M + 255) / 256);
    PanelPlan best{tm, (int)((N + 255) / 256), 0, 0};
    double best_end = makespan(best.tiles_m * best.wide_cols, 1.0, 0, 0.0);
    for (int cn = 1; (int64_t)192 * (cn - 1) < N; cn++) {
        const int64_t left = N - (int64_t)192 * cn;
        const int cw = left > 0 ? (int)((left + 255) / 256) : 0;
        const double end = makespan(tm * cw, 1.0, tm * cn, narrow_cost);
        if (end < best_end - 1e-9) {
            best_end = end;
            best = PanelPlan{tm, cw, cn, 0};
        }
    }
    const int tl = (int)((M + 127) / 128), cl = (int)((N + 255) / 256);
    const double low_end = makespan(tl * cl, low_cost, 0, 0.0);
    if (low_end < best_end - 1e-9) {
        best_end = low_end;
        best = PanelPlan{tl, cl, 0, 1};
    }
    *out = best;
    return best_end;
}

}  // namespace mimir
