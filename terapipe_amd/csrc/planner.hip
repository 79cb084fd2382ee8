// Dynamic-programming slice planner (host code only): the `planning` routine of the reference's
// latency_model.py:97-152, which picks, for a grid of measured single-stage latencies, the batch groups
// and the sequence slices of each group that minimise  sum of slice latencies + (pipeline_len - 1) * largest
// slice latency, subject to every slice latency <= max_latency.
#include "common.h"

#include <cmath>
#include <limits>
#include <vector>

extern "C" int tp_plan_slices(const double* latency_grid, int total_batch_size, int n_steps, int pipeline_len,
                              double max_latency, double* final_time, int* n_groups, int* group_batch,
                              int* group_nslices, int* slice_steps) {
    using tp::set_error;
    if (!latency_grid || !final_time || !n_groups || !group_batch || !group_nslices || !slice_steps) { set_error("tp_plan_slices: null pointer"); return TP_ERR_ARG; }
    if (total_batch_size <= 0 || n_steps <= 0 || pipeline_len <= 0) { set_error("tp_plan_slices: bad sizes B=%d steps=%d pipeline=%d", total_batch_size, n_steps, pipeline_len); return TP_ERR_ARG; }
    const int B = total_batch_size, N = n_steps;
    const double inf = std::numeric_limits<double>::infinity();
    auto grid = [&](int bs, int step, int ctx) { return latency_grid[((size_t)bs * (N + 1) + step) * (N + 1) + ctx]; };
    const size_t W = (size_t)N + 1;
    // f[bs][acc]: best total latency of `acc` steps of sequence at batch size bs (latency_model.py:101-116)
    std::vector<double> f((B + 1) * W, 0.0), fmax((B + 1) * W, 0.0);
    std::vector<long> fstep((B + 1) * W, 0);
    for (int bs = 1; bs <= B; ++bs) {
        for (int acc = 1; acc <= N; ++acc) {
            double best = inf;
            for (int step = 1; step <= acc; ++step) {
                const double lat = grid(bs, step, acc - step);
                const double tot = f[bs * W + acc - step] + lat;
                if (lat <= max_latency && tot < best) {
                    best = tot;
                    fstep[bs * W + acc] = step;
                    fmax[bs * W + acc] = std::fmax(fmax[bs * W + acc - step], lat);
                }
            }
            f[bs * W + acc] = best;
        }
    }
    // g[acc_bs]: best total latency of acc_bs sequences cut into batch groups (:121-133)
    std::vector<double> g(B + 1, 0.0), gmax(B + 1, 0.0);
    std::vector<long> gstep(B + 1, 0);
    for (int acc = 1; acc <= B; ++acc) {
        double best = inf;
        for (int bs = 1; bs <= acc; ++bs) {
            const double tot = g[acc - bs] + f[bs * W + N];
            if (tot < best) {
                best = tot;
                gstep[acc] = bs;
                gmax[acc] = std::fmax(gmax[acc - bs], fmax[bs * W + N]);
            }
        }
        g[acc] = best;
    }
    *final_time = (pipeline_len - 1) * gmax[B] + g[B];                    // :135
    *n_groups = 0;
    if (std::isinf(*final_time) || std::isnan(*final_time)) { *final_time = inf; return TP_OK; }   // no feasible plan (:136-137)
    int cur_b = B, ng = 0, pos = 0;
    while (cur_b > 0) {                                                   // :138-150
        const int bs = (int)gstep[cur_b];
        int cur = N, ns = 0;
        while (cur > 0) {
            const int st = (int)fstep[bs * W + cur];
            slice_steps[pos++] = st;                                      // last slice of the sequence first, as the reference
            cur -= st;
            ++ns;
        }
        group_batch[ng] = bs;
        group_nslices[ng] = ns;
        ++ng;
        cur_b -= bs;
    }
    *n_groups = ng;
    return TP_OK;
}
