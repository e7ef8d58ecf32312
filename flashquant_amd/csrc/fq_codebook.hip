// Lloyd-Max codebook for the coordinates of a rotated unit vector, host code only.
//
// The solver the Python layer of the reference runs at set-up
// (_gaussian_centroids_boundaries, src/flashquant/core/codebook.py:58-140): the coordinates
// are modelled as N(0, 1/dim) truncated to +-3.5 sigma; starting from uniformly spaced
// levels, boundaries (midpoints of neighbouring levels) and levels (conditional means of
// their cells) are updated in turn, in double precision, for at most 200 sweeps or until no
// level moves by 1e-10.  The C++ solver of the reference (csrc/core/codebook.cpp:64-121)
// integrates numerically and gives slightly different levels; the Python one defines the
// values every kernel test uses, so that is the one followed here.
#include <cmath>
#include <vector>

#include "../../include/fq_hip.h"

extern "C" int fq_lloyd_max_gaussian(int dim, int bits, float* centroids, float* boundaries) {
    if (dim <= 0 || bits < 1 || bits > 8) return FQ_ERR_BAD_SHAPE;
    if (!centroids || !boundaries) return FQ_ERR_NULL_POINTER;
    const int levels = 1 << bits;
    const double sigma = 1.0 / std::sqrt(double(dim));
    const double lo = -3.5 * sigma, hi = 3.5 * sigma;
    const double inv_sigma = 1.0 / sigma;
    const double erf_scale = inv_sigma / std::sqrt(2.0);
    const double pdf_scale = 1.0 / (sigma * std::sqrt(2.0 * M_PI));
    auto pdf = [&](double t) { const double z = t * inv_sigma; return pdf_scale * std::exp(-0.5 * z * z); };
    auto cdf = [&](double t) { return 0.5 * (1.0 + std::erf(t * erf_scale)); };

    std::vector<double> c(levels), next(levels), edge(levels + 1);
    for (int i = 0; i < levels; ++i) c[i] = lo + (hi - lo) * (i + 0.5) / levels;
    for (int sweep = 0; sweep < 200; ++sweep) {
        edge[0] = lo;
        edge[levels] = hi;
        for (int i = 1; i < levels; ++i) edge[i] = (c[i - 1] + c[i]) / 2.0;
        double shift = 0.0;
        for (int i = 0; i < levels; ++i) {
            const double a = edge[i], b = edge[i + 1];
            const double mass = cdf(b) - cdf(a);
            next[i] = mass > 1e-15 ? sigma * sigma * (pdf(a) - pdf(b)) / mass : (a + b) / 2.0;
            shift = std::fmax(shift, std::fabs(next[i] - c[i]));
        }
        c.swap(next);
        if (shift < 1e-10) break;
    }
    for (int i = 0; i < levels; ++i) centroids[i] = float(c[i]);
    for (int i = 0; i + 1 < levels; ++i) boundaries[i] = float((c[i] + c[i + 1]) / 2.0);
    return FQ_OK;
}
