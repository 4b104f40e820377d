// Model-file loader: symmetrix JSON -> HostModel.  See smx_host_model.hpp.
#include "smx_host_model.hpp"
#include "smx_poly_tables.inc"

#include <algorithm>
#include <cmath>
#include <fstream>
#include <map>
#include <sstream>
#include <stdexcept>
#include <tuple>

#include "smx_json.hpp"

namespace smx {

namespace {

[[noreturn]] void unsupported(const std::string& what) { throw std::runtime_error("unsupported: " + what); }

// Coefficient table of a spline set, the layout of the reference constructor
// (libsymmetrix/source/cubic_spline_set.cpp:5-25): c[(4*i+q)*nspl + j].
std::vector<double> build_spline_set(double h, const Json& values, const Json& derivs, int& nspl, int& nodes)
{
    nspl = (int)values.size();
    if (nspl == 0 || derivs.size() != (size_t)nspl) throw JsonError("model file: radial spline arrays are empty or differ in size");
    nodes = (int)values[0].size();
    if (nodes < 2) throw JsonError("model file: radial splines need at least two knots");
    std::vector<double> c((size_t)4 * nspl * (nodes - 1));
    for (int j = 0; j < nspl; ++j) {
        const auto& v = values[j].nums;
        const auto& d = derivs[j].nums;
        if (values[j].type != Json::NumArray || derivs[j].type != Json::NumArray ||
            (int)v.size() != nodes || (int)d.size() != nodes)
            throw JsonError("model file: ragged radial spline table");
        for (int i = 0; i < nodes - 1; ++i) {
            c[(size_t)(4 * i) * nspl + j] = v[i];
            c[(size_t)(4 * i + 1) * nspl + j] = d[i];
            c[(size_t)(4 * i + 2) * nspl + j] = (-3 * v[i] - 2 * h * d[i] + 3 * v[i + 1] - h * d[i + 1]) / (h * h);
            c[(size_t)(4 * i + 3) * nspl + j] = (2 * v[i] + h * d[i] - 2 * v[i + 1] + h * d[i + 1]) / (h * h * h);
        }
    }
    return c;
}

void load_radial(const Json& file, const char* vkey, const char* dkey, double h, int expect_pairs,
                 std::vector<int>& pair_table, std::vector<std::vector<double>>& tables, int& nspl, int& nodes)
{
    const Json& V = file.at(vkey);
    const Json& D = file.at(dkey);
    if ((int)V.size() != expect_pairs || (int)D.size() != expect_pairs)
        throw JsonError(std::string("model file: '") + vkey + "' must hold one table per unordered species pair");
    pair_table.assign(expect_pairs, -1);
    nspl = nodes = 0;
    for (int p = 0; p < expect_pairs; ++p) {
        int ns, nn;
        std::vector<double> c = build_spline_set(h, V[p], D[p], ns, nn);
        if (p == 0) { nspl = ns; nodes = nn; }
        else if (ns != nspl || nn != nodes) throw JsonError("model file: radial tables of different pairs differ in shape");
        int found = -1;
        for (size_t u = 0; u < tables.size(); ++u)
            if (tables[u] == c) { found = (int)u; break; }
        if (found < 0) { tables.push_back(std::move(c)); found = (int)tables.size() - 1; }
        pair_table[p] = found;
    }
}

// Single spline coefficients, libsymmetrix/source/cubic_spline.cpp:58-71
std::vector<double> build_splines(double h, const Json& values, const Json& derivs, int& nodes)
{
    const int np = (int)values.size();
    nodes = np ? (int)values[0].size() : 0;
    std::vector<double> c((size_t)np * std::max(0, nodes - 1) * 4);
    for (int p = 0; p < np; ++p) {
        const auto& v = values[p].nums;
        const auto& d = derivs[p].nums;
        if ((int)v.size() != nodes || (int)d.size() != nodes) throw JsonError("model file: ragged density spline table");
        for (int i = 0; i < nodes - 1; ++i) {
            double* ci = c.data() + ((size_t)p * (nodes - 1) + i) * 4;
            ci[0] = v[i];
            ci[1] = d[i];
            ci[2] = (-3 * ci[0] - 2 * h * ci[1] + 3 * v[i + 1] - h * d[i + 1]) / (h * h);
            ci[3] = (2 * ci[0] + h * ci[1] - 2 * v[i + 1] + h * d[i + 1]) / (h * h * h);
        }
    }
    return c;
}

// monomials (each a list of variable indices) + per-(type,k) coefficient lists
// -> rows sharing the first two factors.  Duplicate monomials keep the first
// coefficient, as the std::map::insert of multivariate_polynomial.cpp:36-38.
template <typename CoefFn>
PolySpec build_poly(int num_lm, int T, int K, const std::vector<std::vector<int>>& monomials, CoefFn coef_of, int canon_table)
{
    constexpr int ONE = 16;
    struct Ent { int i0, i1, c, src; };
    std::vector<Ent> ents;
    std::map<std::vector<int>, int> seen;
    for (size_t mi = 0; mi < monomials.size(); ++mi) {
        std::vector<int> mono = monomials[mi];
        if (seen.count(mono)) continue;  // unsorted key, exactly as the reference's map
        seen[mono] = (int)mi;
        if (mono.empty() || mono.size() > 3)
            unsupported("symmetric-contraction monomial of degree " + std::to_string(mono.size()) +
                        " (the device kernels implement degrees 1..3)");
        for (int v : mono)
            if (v < 0 || v >= num_lm) throw JsonError("model file: monomial variable index out of range");
        std::sort(mono.begin(), mono.end());
        Ent e;
        e.src = (int)mi;
        if (mono.size() == 1) { e.i0 = ONE; e.i1 = ONE; e.c = mono[0]; }
        else if (mono.size() == 2) { e.i0 = ONE; e.i1 = mono[0]; e.c = mono[1]; }
        else { e.i0 = mono[0]; e.i1 = mono[1]; e.c = mono[2]; }
        ents.push_back(e);
    }
    // rows of the constant first (degree 1, then degree 2), then degree 3
    auto key = [](const Ent& e) { return std::make_tuple(e.i0 == ONE ? -1 : e.i0, e.i1 == ONE ? -1 : e.i1, e.c); };
    std::stable_sort(ents.begin(), ents.end(), [&](const Ent& a, const Ent& b) { return key(a) < key(b); });
    PolySpec P;
    P.num_entries = (int)ents.size();
    for (size_t i = 0; i < ents.size(); ++i) {
        if (i == 0 || ents[i].i0 != ents[i - 1].i0 || ents[i].i1 != ents[i - 1].i1) {
            P.row_i0.push_back(ents[i].i0);
            P.row_i1.push_back(ents[i].i1);
            P.row_start.push_back((int)i);
        }
        P.entry_var.push_back(ents[i].c);
    }
    P.row_start.push_back((int)ents.size());
    {
        struct LE { int fa, fb, mono, first; };
        std::vector<std::vector<LE>> lists(16);
        for (size_t i = 0; i < ents.size(); ++i) {
            const int f[3] = {ents[i].i0, ents[i].i1, ents[i].c};   // padded with ONE in front
            bool first_done = false;
            for (int pos = 0; pos < 3; ++pos) {
                if (f[pos] == ONE) continue;
                const int fa = f[(pos + 1) % 3], fb = f[(pos + 2) % 3];
                const int is_first = first_done ? 0 : 1;
                first_done = true;
                lists[f[pos]].push_back(LE{fa, fb, (int)i, is_first});
            }
        }
        P.list_start.assign(1, 0);
        for (int v = 0; v < 16; ++v) {
            std::stable_sort(lists[v].begin(), lists[v].end(), [](const LE& a, const LE& b) { return a.first > b.first; });
            int nf = 0;
            for (auto& e : lists[v]) {
                nf += e.first;
                P.list_fa.push_back(e.fa); P.list_fb.push_back(e.fb); P.list_mono.push_back(e.mono);
            }
            P.list_nfirst.push_back(nf);
            P.list_start.push_back((int)P.list_fa.size());
        }
        if (ents.size() >= 65535) unsupported("more than 65534 monomials in one symmetric-contraction polynomial");
        const int dummy = (int)ents.size() | (ONE << 16) | (ONE << 24);
        // variables in the order the wavefront groups walk them: group g owns v = g, g + POLY_GROUPS, ...
        for (int g = 0; g < POLY_GROUPS; ++g)
            for (int v = g; v < 16; v += POLY_GROUPS) {
                const int s0 = P.list_start[v], sf = s0 + P.list_nfirst[v], s1 = P.list_start[v + 1];
                const int bounds[3] = {s0, sf, s1};
                for (int part = 0; part < 2; ++part) {
                    int n = 0;
                    for (int e = bounds[part]; e < bounds[part + 1]; ++e, ++n)
                        P.packed.push_back(P.list_mono[e] | (P.list_fa[e] << 16) | (P.list_fb[e] << 24));
                    while (n % 4) { P.packed.push_back(dummy); ++n; }
                    P.chunks.push_back(n / 4);
                }
            }
        for (int q = 0; q < 4 * POLY_SPARE_CHUNKS; ++q) P.packed.push_back(dummy);
    }
    // one extra all-zero coefficient row per species for the padding entries
    P.coef.assign((size_t)T * (ents.size() + 1) * K, 0.0);
    for (int a = 0; a < T; ++a)
        for (int k = 0; k < K; ++k) {
            const std::vector<double>& w = coef_of(a, k);
            if (w.size() != monomials.size()) throw JsonError("model file: polynomial weights and monomials differ in length");
            for (size_t i = 0; i < ents.size(); ++i)
                P.coef[((size_t)a * (ents.size() + 1) + i) * K + k] = w[ents[i].src];
        }
    // the standard product basis: every monomial of the file inside the compile-time table of this output slot?
    int tn = 0;
    const unsigned char (*tab)[3] = poly_table(canon_table, &tn);
    if (tab) {
        std::map<std::tuple<int, int, int>, int> where;
        for (int i = 0; i < tn; ++i) where[std::make_tuple((int)tab[i][0], (int)tab[i][1], (int)tab[i][2])] = i;
        std::vector<int> slot(ents.size(), -1);
        bool inside = true;
        for (size_t i = 0; i < ents.size() && inside; ++i) {
            auto it = where.find(std::make_tuple(ents[i].i0, ents[i].i1, ents[i].c));
            if (it == where.end()) inside = false;
            else slot[i] = it->second;
        }
        if (inside) {
            P.table = canon_table;
            P.table_coef.assign((size_t)T * tn * K, 0.0);
            for (int a = 0; a < T; ++a)
                for (int k = 0; k < K; ++k) {
                    const std::vector<double>& w = coef_of(a, k);
                    for (size_t i = 0; i < ents.size(); ++i)
                        P.table_coef[((size_t)a * tn + slot[i]) * K + k] = w[ents[i].src];
                }
        }
    }
    return P;
}

std::vector<std::vector<int>> monomial_list(const Json& j)
{
    std::vector<std::vector<int>> out;
    if (j.type == Json::Array) {
        for (const auto& e : j.arr) out.push_back(e.as_ints());
    } else if (j.type == Json::NumArray) {
        unsupported("monomial list is flat");
    }
    return out;
}

}  // namespace

HostModel load_host_model(const std::string& path)
{
    std::ifstream f(path, std::ios::binary);
    if (!f) throw JsonError("model file: cannot open '" + path + "'");
    std::stringstream ss;
    ss << f.rdbuf();
    const std::string text = ss.str();
    Json file = JsonParser(text).parse();
    if (file.type != Json::Object) throw JsonError("model file: top level is not an object");

    HostModel m;
    // basic information, mace.cpp:912-920
    m.T = file.at("num_elements").as_int();
    m.K = file.at("num_channels").as_int();
    m.r_cut = file.at("r_cut").as_double();
    m.l_max = file.at("l_max").as_int();
    m.num_lm = (m.l_max + 1) * (m.l_max + 1);
    m.L_max = file.at("L_max").as_int();
    m.num_LM = (m.L_max + 1) * (m.L_max + 1);
    m.atomic_numbers = file.at("atomic_numbers").as_ints();
    m.atomic_energies = file.at("atomic_energies").as_doubles();
    const int T = m.T, K = m.K;
    if (T <= 0 || K <= 0) throw JsonError("model file: num_elements and num_channels must be positive");
    if ((int)m.atomic_numbers.size() != T || (int)m.atomic_energies.size() != T)
        throw JsonError("model file: atomic_numbers/atomic_energies do not have num_elements entries");
    if (m.l_max != 3) unsupported("l_max = " + std::to_string(m.l_max) + " (the harmonics kernels implement l_max = 3, as the reference's extractor requires)");
    if (m.L_max < 0 || m.L_max > 2) unsupported("L_max = " + std::to_string(m.L_max) + " (device kernels exist for hidden features up to L_max = 2)");

    // ZBL, mace.cpp:922-930
    m.has_zbl = file.at("has_zbl").as_bool();
    if (m.has_zbl) {
        m.zbl_a_exp = file.at("zbl_a_exp").as_double();
        m.zbl_a_prefactor = file.at("zbl_a_prefactor").as_double();
        m.zbl_c = file.at("zbl_c").as_doubles();
        m.zbl_covalent_radii = file.at("zbl_covalent_radii").as_doubles();
        m.zbl_p = file.at("zbl_p").as_int();
        if (m.zbl_c.size() != 4) throw JsonError("model file: zbl_c must have four entries");
    }

    // radial splines, mace.cpp:932-941
    m.spl_h = file.at("radial_spline_h").as_double();
    m.num_pairs = T * (T + 1) / 2;
    int nodes1 = 0;
    load_radial(file, "radial_spline_values_0", "radial_spline_derivs_0", m.spl_h, m.num_pairs,
                m.pair_table0, m.tables0, m.nspl0, m.spl_nodes);
    load_radial(file, "radial_spline_values_1", "radial_spline_derivs_1", m.spl_h, m.num_pairs,
                m.pair_table1, m.tables1, m.nspl1, nodes1);
    if (nodes1 != m.spl_nodes) throw JsonError("model file: layer-0 and layer-1 radial tables differ in knot count");
    if (m.nspl0 != (m.l_max + 1) * K) throw JsonError("model file: radial_spline_values_0 must hold (l_max+1)*num_channels functions");

    m.H0_weights = file.at("H0_weights").as_doubles();
    if ((int)m.H0_weights.size() != T * K) throw JsonError("model file: H0_weights must have num_elements*num_channels entries");

    // A0 weights [T][l][K*K], mace.cpp:947
    {
        const Json& A = file.at("A0_weights");
        if ((int)A.size() != T) throw JsonError("model file: A0_weights must have one block per element");
        m.A0_weights.reserve((size_t)T * (m.l_max + 1) * K * K);
        for (int a = 0; a < T; ++a) {
            if ((int)A[a].size() != m.l_max + 1) throw JsonError("model file: A0_weights[a] must have l_max+1 blocks");
            for (int l = 0; l <= m.l_max; ++l) {
                const auto& w = A[a][l].nums;
                if ((int)w.size() != K * K) throw JsonError("model file: A0_weights block is not K*K");
                m.A0_weights.insert(m.A0_weights.end(), w.begin(), w.end());
            }
        }
    }
    // density normalisation, mace.cpp:949-957 and 994-1002
    m.A0_scaled = file.at("A0_scaled").as_bool();
    if (m.A0_scaled) {
        m.A0_spline_h = file.at("A0_spline_h").as_double();
        m.A0_spline_c = build_splines(m.A0_spline_h, file.at("A0_spline_values"), file.at("A0_spline_derivs"), m.A0_spline_nodes);
    }
    m.A1_scaled = file.at("A1_scaled").as_bool();
    if (m.A1_scaled) {
        m.A1_spline_h = file.at("A1_spline_h").as_double();
        m.A1_spline_c = build_splines(m.A1_spline_h, file.at("A1_spline_values"), file.at("A1_spline_derivs"), m.A1_spline_nodes);
    }

    // M0, mace.cpp:959-972
    {
        const Json& W = file.at("M0_weights");
        const Json& M = file.at("M0_monomials");
        m.P0.resize(m.num_LM);
        for (int LM = 0; LM < m.num_LM; ++LM) {
            auto monos = monomial_list(M.at(std::to_string(LM)));
            m.P0[LM] = build_poly(m.num_lm, T, K, monos, [&](int a, int k) -> const std::vector<double>& {
                return W.at(std::to_string(a)).at(std::to_string(LM)).at(std::to_string(k)).nums;
            }, LM);
        }
    }
    m.H1_weights = file.at("H1_weights").as_doubles();
    if ((int)m.H1_weights.size() != (m.L_max + 1) * K * K) throw JsonError("model file: H1_weights must have (L_max+1)*K*K entries");

    // Phi1, mace.cpp:977-989
    m.Phi1_l = file.at("Phi1_l").as_ints();
    m.Phi1_l1 = file.at("Phi1_l1").as_ints();
    m.Phi1_l2 = file.at("Phi1_l2").as_ints();
    m.Phi1_lme = file.at("Phi1_lme").as_ints();
    m.Phi1_cg = file.at("Phi1_clebsch_gordan").as_doubles();
    m.Phi1_lelm1lm2 = file.at("Phi1_lelm1lm2").as_ints();
    m.num_paths = (int)m.Phi1_l.size();
    if ((int)m.Phi1_l1.size() != m.num_paths || (int)m.Phi1_l2.size() != m.num_paths)
        throw JsonError("model file: Phi1_l, Phi1_l1, Phi1_l2 differ in length");
    if (m.Phi1_lme.size() != m.Phi1_cg.size() || m.Phi1_lelm1lm2.size() != m.Phi1_cg.size())
        throw JsonError("model file: Phi1_lme, Phi1_clebsch_gordan, Phi1_lelm1lm2 differ in length");
    {
        // canonical enumeration for this L_max (see smx_paths.hpp)
        std::vector<std::tuple<int, int, int>> canon;
        for (int l = 0; l <= m.l_max; ++l)
            for (int l2 = 0; l2 <= m.L_max; ++l2)
                for (int l1 = 0; l1 <= m.l_max; ++l1)
                    if (std::abs(l1 - l2) <= l && l <= l1 + l2 && (l + l1 + l2) % 2 == 0) canon.emplace_back(l, l1, l2);
        bool same = (int)canon.size() == m.num_paths;
        for (int p = 0; same && p < m.num_paths; ++p)
            same = canon[p] == std::make_tuple(m.Phi1_l[p], m.Phi1_l1[p], m.Phi1_l2[p]);
        if (!same) unsupported("layer-1 tensor-product path list differs from the full parity-allowed list sorted by output order");
    }
    m.num_e.assign(m.l_max + 1, 0);
    m.num_lme = 0;
    m.num_lelm1lm2 = 0;
    std::vector<int> qoff(m.num_paths + 1, 0), boff(m.num_paths + 1, 0), e_of(m.num_paths, 0);
    for (int p = 0; p < m.num_paths; ++p) {
        e_of[p] = m.num_e[m.Phi1_l[p]];
        m.num_e[m.Phi1_l[p]] += 1;
        m.num_lme += 2 * m.Phi1_l[p] + 1;
        qoff[p + 1] = qoff[p] + (2 * m.Phi1_l1[p] + 1) * (2 * m.Phi1_l2[p] + 1);
        boff[p + 1] = boff[p] + (2 * m.Phi1_l[p] + 1) * (2 * m.Phi1_l2[p] + 1);
    }
    m.num_lelm1lm2 = qoff[m.num_paths];
    m.num_B = boff[m.num_paths];
    {
        std::vector<int> lme_off(m.l_max + 2, 0);
        for (int l = 0; l <= m.l_max; ++l) lme_off[l + 1] = lme_off[l] + (2 * l + 1) * m.num_e[l];
        std::vector<std::vector<std::pair<int, double>>> rows(m.num_B);
        for (size_t c = 0; c < m.Phi1_cg.size(); ++c) {
            const int lme = m.Phi1_lme[c], q = m.Phi1_lelm1lm2[c];
            if (lme < 0 || lme >= m.num_lme || q < 0 || q >= m.num_lelm1lm2)
                throw JsonError("model file: Clebsch-Gordan index out of range");
            int p = 0;
            while (q >= qoff[p + 1]) ++p;
            const int l2 = m.Phi1_l2[p], l1 = m.Phi1_l1[p];
            const int m1 = (q - qoff[p]) / (2 * l2 + 1), m2 = (q - qoff[p]) % (2 * l2 + 1);
            int l = 0;
            while (lme >= lme_off[l + 1]) ++l;
            const int mm = (lme - lme_off[l]) / m.num_e[l], e = (lme - lme_off[l]) % m.num_e[l];
            if (l != m.Phi1_l[p] || e != e_of[p])
                unsupported("a Clebsch-Gordan entry couples a product of one path into the output slot of another path");
            rows[boff[p] + mm * (2 * l2 + 1) + m2].emplace_back(l1 * l1 + m1, m.Phi1_cg[c]);
        }
        m.B_start.assign(1, 0);
        for (int b = 0; b < m.num_B; ++b) {
            for (auto& pr : rows[b]) { m.B_lm1.push_back(pr.first); m.B_c.push_back(pr.second); }
            m.B_start.push_back((int)m.B_lm1.size());
        }
    }
    if (m.nspl1 != m.num_paths * K) throw JsonError("model file: radial_spline_values_1 must hold num_paths*num_channels functions");

    // A1 weights per l, mace.cpp:992
    {
        const Json& A = file.at("A1_weights");
        if ((int)A.size() != m.l_max + 1) throw JsonError("model file: A1_weights must have l_max+1 blocks");
        for (int l = 0; l <= m.l_max; ++l) {
            auto w = A[l].as_doubles();
            if ((int)w.size() != m.num_e[l] * K * K) throw JsonError("model file: A1_weights block has the wrong size");
            m.A1_weights.push_back(std::move(w));
        }
    }
    // M1, mace.cpp:1004-1015
    {
        const Json& W = file.at("M1_weights");
        auto monos = monomial_list(file.at("M1_monomials"));
        m.P1 = build_poly(m.num_lm, T, K, monos, [&](int a, int k) -> const std::vector<double>& {
            return W.at(std::to_string(a)).at(std::to_string(k)).nums;
        }, 0);
    }
    // H2 and readouts, mace.cpp:1017-1029
    {
        const Json& A = file.at("H2_weights_for_H1");
        if ((int)A.size() != T) throw JsonError("model file: H2_weights_for_H1 must have one block per element");
        for (int a = 0; a < T; ++a) {
            auto w = A[a].as_doubles();
            if ((int)w.size() != K * K) throw JsonError("model file: H2_weights_for_H1 block is not K*K");
            m.H2_weights_for_H1.insert(m.H2_weights_for_H1.end(), w.begin(), w.end());
        }
    }
    m.H2_weights_for_M1 = file.at("H2_weights_for_M1").as_doubles();
    if ((int)m.H2_weights_for_M1.size() != K * K) throw JsonError("model file: H2_weights_for_M1 is not K*K");
    m.readout_1_weights = file.at("readout_1_weights").as_doubles();
    m.readout_2_w1 = file.at("readout_2_weights_1").as_doubles();
    m.readout_2_w2 = file.at("readout_2_weights_2").as_doubles();
    m.readout_2_scale = file.at("readout_2_scale_factor").as_double();
    if ((int)m.readout_1_weights.size() != K || (int)m.readout_2_w1.size() != 16 * K || (int)m.readout_2_w2.size() != 16)
        throw JsonError("model file: readout weights have the wrong size (hidden width is fixed at 16, mace.cpp:1022-1029)");
    return m;
}

}  // namespace smx
