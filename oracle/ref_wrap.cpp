// C-ABI shim over the few reference translation units that compile from their
// own sources with no third-party dependency (cubic_spline_set.cpp,
// cubic_spline.cpp, tools.cpp, zbl.cpp under libsymmetrix/source).  Built only
// in a container that has the reference tree, into oracle/_ref/ (git-ignored);
// used by the tests to validate the C restatement in mace_oracle.c.  The rest of
// the reference (mace.cpp, multivariate_polynomial.cpp,
// multilayer_perceptron.cpp) needs sphericart, a CBLAS header and
// nlohmann/json, none of which the tree or the image provides, so it is not
// built.
#include <vector>
#include <cstring>
#include <stdexcept>

#include "cubic_spline.hpp"
#include "cubic_spline_set.hpp"
#include "tools.hpp"
#include "zbl.hpp"

extern "C" {

// flattened result: for each partition, len(part0), part0..., len(part1), part1...
int ref_two_part_partitions(const int* v, int n, int* out, int cap)
{
    auto parts = _two_part_partitions(std::vector<int>(v, v + n));
    int pos = 0, count = 0;
    for (auto& p : parts) {
        for (auto& s : p) {
            if (pos + 1 + (int)s.size() > cap) return -1;
            out[pos++] = (int)s.size();
            for (int x : s) out[pos++] = x;
        }
        count += 1;
    }
    return count;
}

int ref_num_partitions(int n)
{
    std::vector<int> v(n);
    for (int i = 0; i < n; ++i) v[i] = i;
    return (int)_partitions(v).size();
}

void* ref_spline_set_create(double h, int num_splines, int num_nodes, const double* values, const double* derivs)
{
    std::vector<std::vector<double>> v(num_splines), d(num_splines);
    for (int j = 0; j < num_splines; ++j) {
        v[j].assign(values + (size_t)j * num_nodes, values + (size_t)(j + 1) * num_nodes);
        d[j].assign(derivs + (size_t)j * num_nodes, derivs + (size_t)(j + 1) * num_nodes);
    }
    return new CubicSplineSet(h, v, d);
}
void ref_spline_set_evaluate_derivs(void* s, double r, double* values, double* derivs)
{
    auto* set = static_cast<CubicSplineSet*>(s);
    set->evaluate_derivs(r, std::span<double>(values, set->num_splines), std::span<double>(derivs, set->num_splines));
}
void ref_spline_set_evaluate(void* s, double r, double* values)
{
    auto* set = static_cast<CubicSplineSet*>(s);
    set->evaluate(r, std::span<double>(values, set->num_splines));
}
void ref_spline_set_free(void* s) { delete static_cast<CubicSplineSet*>(s); }

void* ref_spline_create(double h, int num_nodes, const double* values, const double* derivs)
{
    return new CubicSpline(h, std::vector<double>(values, values + num_nodes), std::vector<double>(derivs, derivs + num_nodes));
}
int ref_spline_evaluate_deriv(void* s, double r, double* f, double* d)
{
    try {
        auto [ff, dd] = static_cast<CubicSpline*>(s)->evaluate_deriv(r);
        *f = ff; *d = dd;
        return 0;
    } catch (const std::invalid_argument&) {
        return -1;
    }
}
void ref_spline_free(void* s) { delete static_cast<CubicSpline*>(s); }

void* ref_zbl_create(double a_exp, double a_prefactor, const double* c, const double* radii, int n_radii, int p)
{
    return new ZBL(a_exp, a_prefactor, std::vector<double>(c, c + 4), std::vector<double>(radii, radii + n_radii), p);
}
double ref_zbl_compute(void* z, int Zu, int Zv, double r) { return static_cast<ZBL*>(z)->compute(Zu, Zv, r); }
double ref_zbl_compute_gradient(void* z, int Zu, int Zv, double r) { return static_cast<ZBL*>(z)->compute_gradient(Zu, Zv, r); }
double ref_zbl_envelope(void* z, double r, double r_max, int p) { return static_cast<ZBL*>(z)->compute_envelope(r, r_max, p); }
void ref_zbl_compute_ZBL(void* z, int num_nodes, const int* node_types, const int* num_neigh, const int* neigh_types,
                         const int* atomic_numbers, int T, const double* r, const double* xyz, long E,
                         double* node_energies, double* node_forces)
{
    static_cast<ZBL*>(z)->compute_ZBL(num_nodes, std::span<const int>(node_types, num_nodes),
        std::span<const int>(num_neigh, num_nodes), std::span<const int>(neigh_types, E),
        std::span<const int>(atomic_numbers, T), std::span<const double>(r, E), std::span<const double>(xyz, 3 * E),
        std::span<double>(node_energies, num_nodes), std::span<double>(node_forces, 3 * E));
}
void ref_zbl_free(void* z) { delete static_cast<ZBL*>(z); }

}
