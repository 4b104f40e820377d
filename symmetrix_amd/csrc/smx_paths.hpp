// Compile-time description of the layer-1 tensor-product paths.
//
// The model file lists the paths as Phi1_l / Phi1_l1 / Phi1_l2
// (libsymmetrix/source/mace.cpp:978-989): output order l, order l1 of the
// spherical harmonic and order l2 of the sender feature.  The extractor takes
// them from e3nn's instruction list sorted by output irrep
// (symmetrix/source/symmetrix/extract_mace_data.py:323-325), which enumerates
// l2 outer and l1 inner and keeps every coupling allowed by the triangle rule
// and by parity (l + l1 + l2 even for 0e,1o,2e,3o features) with l <= 3.  The
// kernels keep per-path accumulators in registers, so this list is fixed at
// compile time per L_max and checked against the file at load.
#pragma once

namespace smx {

constexpr int kLmaxY = 3;   // order of the edge harmonics (the extractor refuses anything else)
constexpr int kNumLm = 16;

template <int LMAXH>
struct Paths {
    static constexpr int count()
    {
        int n = 0;
        for (int l = 0; l <= kLmaxY; ++l)
            for (int l2 = 0; l2 <= LMAXH; ++l2)
                for (int l1 = 0; l1 <= kLmaxY; ++l1)
                    if (allowed(l, l1, l2)) ++n;
        return n;
    }
    static constexpr bool allowed(int l, int l1, int l2)
    {
        const int lo = l1 > l2 ? l1 - l2 : l2 - l1;
        return lo <= l && l <= l1 + l2 && ((l + l1 + l2) % 2 == 0);
    }
    // which = 0: l, 1: l1, 2: l2 of path p
    static constexpr int get(int p, int which)
    {
        int n = 0;
        for (int l = 0; l <= kLmaxY; ++l)
            for (int l2 = 0; l2 <= LMAXH; ++l2)
                for (int l1 = 0; l1 <= kLmaxY; ++l1)
                    if (allowed(l, l1, l2)) {
                        if (n == p) return which == 0 ? l : (which == 1 ? l1 : l2);
                        ++n;
                    }
        return -1;
    }
    static constexpr int P = count();
    static constexpr int NLM = (LMAXH + 1) * (LMAXH + 1);
    static constexpr int l(int p) { return get(p, 0); }
    static constexpr int l1(int p) { return get(p, 1); }
    static constexpr int l2(int p) { return get(p, 2); }
    static constexpr int num_e(int l_)
    {
        int n = 0;
        for (int p = 0; p < P; ++p) if (l(p) == l_) ++n;
        return n;
    }
    // rank of path p among the paths with the same output order
    static constexpr int e(int p)
    {
        int n = 0;
        for (int q = 0; q < p; ++q) if (l(q) == l(p)) ++n;
        return n;
    }
    static constexpr int lme_off(int l_)
    {
        int n = 0;
        for (int q = 0; q < l_; ++q) n += (2 * q + 1) * num_e(q);
        return n;
    }
    // index into Phi1[lme]: layout [l][m][e], extract_mace_data.py:336-342
    static constexpr int lme(int p, int m) { return lme_off(l(p)) + m * num_e(l(p)) + e(p); }
    static constexpr int NE = lme_off(kLmaxY + 1);
    // offset of path p in the per-edge coupling matrix B[path][m][m2]
    static constexpr int boff(int p)
    {
        int n = 0;
        for (int q = 0; q < p; ++q) n += (2 * l(q) + 1) * (2 * l2(q) + 1);
        return n;
    }
    static constexpr int NB = boff(P);
    // offset of path p in the reference's Phi1r index lelm1lm2, mace.cpp:468-483
    static constexpr int qoff(int p)
    {
        int n = 0;
        for (int q = 0; q < p; ++q) n += (2 * l1(q) + 1) * (2 * l2(q) + 1);
        return n;
    }
};

}  // namespace smx
